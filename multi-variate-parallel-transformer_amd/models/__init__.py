"""Plain torch.nn.Module counterparts of the reference's tag classes (models/__init__.py:1-18)."""
from torch.nn import Module


class BrainModel(Module):
    pass


class PartialModel(Module):
    pass


class BrainEncoder(Module):
    pass


class BrainQuantizer(Module):
    pass


class BrainDecider(Module):
    pass
