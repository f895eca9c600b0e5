from .mvpa import (MvpaKVCache, MvpaRingCache, MvpaRingClock, MVPFormerGQAAttention,
                   MVPFormerGQAFlashAttention)

__all__ = ["MvpaKVCache", "MvpaRingCache", "MvpaRingClock", "MVPFormerGQAAttention",
           "MVPFormerGQAFlashAttention"]
