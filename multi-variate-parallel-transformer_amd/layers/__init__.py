from .mvpa import (KeyMask, MvpaKVCache, MvpaRingCache, MvpaRingClock, MVPFormerGQAAttention,
                   MVPFormerGQAFlashAttention)

__all__ = ["KeyMask", "MvpaKVCache", "MvpaRingCache", "MvpaRingClock", "MVPFormerGQAAttention",
           "MVPFormerGQAFlashAttention"]
