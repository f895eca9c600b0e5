"""Seeded synthetic inputs for the MVPA operator and for the MVPFormer forward.

No dataset or checkpoint ships with this build, so every test and benchmark draws its
inputs here.  All draws happen on the CPU in a fixed order so that a seed names the same
numbers on every machine.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

# The five benchmark configurations (shapes only).
MVPA_CONFIGS = {
    "c1": dict(B=2, C=8, T=32, H=4, Hkv=4, Dh=32, qkv_unit=False),
    "c2": dict(B=4, C=64, T=128, H=16, Hkv=16, Dh=64, qkv_unit=True),
    "c3": dict(B=8, C=117, T=256, H=16, Hkv=16, Dh=64, qkv_unit=True, validity=True),
}


@dataclass
class MvpaInputs:
    q: torch.Tensor        # [B,H,N,Dh]
    k: torch.Tensor        # [B,Hkv,N,Dh]
    v: torch.Tensor        # [B,Hkv,N,Dh]
    k_time: torch.Tensor   # [Hkv,T,Dh]
    k_chan: torch.Tensor   # [Hkv,C,Dh]
    u: torch.Tensor        # [Hkv,Dh]
    vb: torch.Tensor       # [Hkv,Dh]
    z: torch.Tensor        # [Hkv,Dh]
    chan_valid: Optional[torch.Tensor]  # [B,C] bool
    T: int
    C: int

    def to(self, device=None, dtype=None) -> "MvpaInputs":
        def mv(t):
            return t.to(device=device, dtype=dtype) if t is not None else None
        cv = self.chan_valid.to(device=device) if self.chan_valid is not None else None
        return MvpaInputs(mv(self.q), mv(self.k), mv(self.v), mv(self.k_time), mv(self.k_chan),
                          mv(self.u), mv(self.vb), mv(self.z), cv, self.T, self.C)

    def round_to(self, dtype) -> "MvpaInputs":
        """Same values after a round trip through ``dtype`` (still float32)."""
        def rt(t):
            return t.to(dtype).to(torch.float32)
        return MvpaInputs(rt(self.q), rt(self.k), rt(self.v), rt(self.k_time), rt(self.k_chan),
                          rt(self.u), rt(self.vb), rt(self.z), self.chan_valid, self.T, self.C)


def make_mvpa_inputs(B: int, C: int, T: int, H: int, Dh: int, Hkv: Optional[int] = None,
                     seed: int = 0, qkv_unit: bool = False, validity: bool = False,
                     table_std: float = 0.02) -> MvpaInputs:
    """float32 CPU tensors drawn in the order q, k, v, k_time, k_chan, attn_bias, validity.

    q, k, v ~ N(0,1), divided by sqrt(Dh) when ``qkv_unit``; tables and biases ~ N(0, table_std).
    ``validity`` draws a live fraction U(0.7, 1.0) per sample and keeps channel c when
    rand(c) < fraction (at least one channel is always kept).
    """
    Hkv = H if Hkv is None else Hkv
    g = torch.Generator(device="cpu").manual_seed(seed)
    N = T * C
    scale = Dh ** -0.5 if qkv_unit else 1.0
    q = torch.randn((B, H, N, Dh), generator=g) * scale
    k = torch.randn((B, Hkv, N, Dh), generator=g) * scale
    v = torch.randn((B, Hkv, N, Dh), generator=g) * scale
    k_time = torch.randn((Hkv, T, Dh), generator=g) * table_std
    k_chan = torch.randn((Hkv, C, Dh), generator=g) * table_std
    attn_bias = torch.randn((3 * Hkv * Dh,), generator=g) * table_std
    u, vb, z = (t.view(Hkv, Dh) for t in attn_bias.split(Hkv * Dh))
    chan_valid = None
    if validity:
        frac = 0.7 + 0.3 * torch.rand((B,), generator=g)
        chan_valid = torch.rand((B, C), generator=g) < frac[:, None]
        for b in range(B):
            if not chan_valid[b].any():
                chan_valid[b, 0] = True
    return MvpaInputs(q, k, v, k_time, k_chan, u.contiguous(), vb.contiguous(), z.contiguous(),
                      chan_valid, T, C)


def make_ieeg(B: int, C: int, T: int, seg: int = 512, seed: int = 0) -> torch.Tensor:
    """Synthetic iEEG at ``seg`` Hz: per channel 1/f^alpha noise (alpha ~ U(1,2)) plus one to
    three sinusoids at 4-40 Hz, z-scored per channel, cut into T one-second segments.
    Returns float32 [B,T,C,seg]."""
    rng = np.random.default_rng(seed)
    n = T * seg
    freqs = np.fft.rfftfreq(n, d=1.0 / seg)
    t = np.arange(n) / seg
    out = np.empty((B, C, n), dtype=np.float32)
    for b in range(B):
        for c in range(C):
            alpha = rng.uniform(1.0, 2.0)
            spec = np.fft.rfft(rng.standard_normal(n))
            shape = np.zeros_like(freqs)
            shape[1:] = freqs[1:] ** (-alpha / 2.0)
            x = np.fft.irfft(spec * shape, n=n)
            sd = x.std()
            for _ in range(int(rng.integers(1, 4))):
                f = rng.uniform(4.0, 40.0)
                ph = rng.uniform(0.0, 2 * np.pi)
                amp = rng.uniform(0.5, 1.5) * sd
                x = x + amp * np.sin(2 * np.pi * f * t + ph)
            x = (x - x.mean()) / x.std()
            out[b, c] = x.astype(np.float32)
    x = torch.from_numpy(out).view(B, C, T, seg).permute(0, 2, 1, 3).contiguous()
    return x
