"""MVPFormer-S forward throughput (windows per second) on one GPU, for bench.py."""
from __future__ import annotations

import time

import torch

from mvpa_hip.synthetic import make_ieeg
from models.configs import MVPFORMER_S
from models.fftencoder import WaveEncoder
from models.mvpformer import HMVPFormer, MVPFormerConfig, MVPFormerHead


def build_mvpformer_s(seg: int = 512, device="cuda:0", seed: int = 0, n_layer=None, n_positions=None):
    """Random-init MVPFormer-S (E768 L12 H12 Hkv4 n_inner1728) in bf16 with an E->E head for
    next-segment prediction."""
    torch.manual_seed(seed)
    dims = dict(MVPFORMER_S)
    if n_layer is not None:
        dims["n_layer"] = n_layer
    if n_positions is not None:
        dims["n_positions"] = n_positions
    cfg = MVPFormerConfig(**dims)
    model = HMVPFormer(cfg, WaveEncoder(seg, cfg.n_embd), MVPFormerHead(cfg.n_embd, cfg.n_embd))
    return model.to(device=device, dtype=torch.bfloat16).eval()


def mvpformer_s_windows_per_s(B: int = 4, C: int = 64, T: int = 64, seg: int = 512,
                              steps: int = 20, warmup: int = 10) -> dict:
    model = build_mvpformer_s(seg)
    x = make_ieeg(B, C, T, seg, seed=0).to("cuda:0")
    for _ in range(warmup):
        model.predict_next_segment(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        model.predict_next_segment(x)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {"windows_per_s": round(B / (ms * 1e-3), 2), "ms_per_forward": round(ms, 3),
            "config": f"MVPFormer-S E768 L12 H12 Hkv4 Dh64 n_inner1728, B={B} C={C} T={T} "
                      f"segments of {seg} samples, bf16, random-init weights, synthetic iEEG"}
