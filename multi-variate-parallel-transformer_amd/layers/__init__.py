from .mvpa import MvpaKVCache, MvpaRingCache, MVPFormerGQAAttention, MVPFormerGQAFlashAttention

__all__ = ["MvpaKVCache", "MvpaRingCache", "MVPFormerGQAAttention", "MVPFormerGQAFlashAttention"]
