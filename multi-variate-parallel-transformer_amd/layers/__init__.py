from .mvpa import MVPFormerGQAAttention, MVPFormerGQAFlashAttention

__all__ = ["MVPFormerGQAAttention", "MVPFormerGQAFlashAttention"]
