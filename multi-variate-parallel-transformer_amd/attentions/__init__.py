from .attn import flash_mvpa as flashmvpa
from .attn import flash_mvpa

__all__ = ["flashmvpa", "flash_mvpa"]
