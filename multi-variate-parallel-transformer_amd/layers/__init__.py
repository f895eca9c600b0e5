from .mvpa import MvpaKVCache, MVPFormerGQAAttention, MVPFormerGQAFlashAttention

__all__ = ["MvpaKVCache", "MVPFormerGQAAttention", "MVPFormerGQAFlashAttention"]
