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


def mvpformer_s_stream_step_ms(C: int = 64, T: int = 64, seg: int = 512, steps: int = 40) -> dict:
    """One window of C channels as a stream: the steady-state cost of one new segment
    (classify_step: encoder on the segment, one decoding step per block against caches holding the
    last T segments) beside the full forward over the same T segments."""
    model = build_mvpformer_s(seg, n_positions=T)
    x = make_ieeg(1, C, T + steps, seg, seed=1).to("cuda:0")
    past = None
    for t in range(T):                       # fill the window; the caches slide from here on
        _, past = model.classify_step(x[:, t], past)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(T, T + steps):
        _, past = model.classify_step(x[:, t], past)
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) * 1e3 / steps
    # the same step on ring caches, replayed as one HIP graph
    graph_step = model.capture_stream(past, x[:, 0])
    for t in range(5):
        graph_step(x[:, t])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(steps):
        graph_step(x[:, T + t])
    torch.cuda.synchronize()
    graph_ms = (time.perf_counter() - t0) * 1e3 / steps
    for _ in range(5):
        model.classify(x[:, :T])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        model.classify(x[:, :T])
    torch.cuda.synchronize()
    full_ms = (time.perf_counter() - t0) * 1e3 / 10
    return {"ms_per_segment": round(step_ms, 3), "ms_per_segment_graph_replay": round(graph_ms, 3),
            "ms_full_forward_same_window": round(full_ms, 3),
            "config": f"MVPFormer-S, B=1 C={C}, window of {T} segments of {seg} samples, bf16"}


def mvpformer_base_forward_ms(C: int = 128, T: int = 512, seg: int = 512, steps: int = 3,
                              warmup: int = 2, stream: bool = True) -> dict:
    """Random-init base-size classification forward (E2048 L24 H16 Hkv8 Dh128 n_inner5632, binary
    head) on one window of C channels x T segments: bf16, then fp8 e4m3 QK^T."""
    from models.configs import MVPFORMER_BASE
    x = make_ieeg(1, C, T, seg, seed=7).to("cuda:0")
    res = {"config": f"MVPFormer base E2048 L24 H16 Hkv8 Dh128 n_inner5632 + binary head, B=1 C={C} "
                     f"T={T} segments of {seg} samples, random-init weights, synthetic iEEG"}
    logits = {}
    for fp8 in (False, True):
        torch.manual_seed(3)
        cfg = MVPFormerConfig(**dict(MVPFORMER_BASE, n_positions=max(T, 110)), fp8_qk=fp8)
        model = HMVPFormer(cfg, WaveEncoder(seg, cfg.n_embd), MVPFormerHead(cfg.n_embd, 2))
        model = model.to(device="cuda:0", dtype=torch.bfloat16).eval()
        for _ in range(warmup):
            y = model.classify(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            y = model.classify(x)
        torch.cuda.synchronize()
        res["ms_per_forward_fp8_qk" if fp8 else "ms_per_forward_bf16"] = round(
            (time.perf_counter() - t0) * 1e3 / steps, 1)
        logits[fp8] = y.float().cpu()
        if not fp8 and stream:
            # the same window as a stream: fill the caches, then time segments that slide it
            past = None
            for t in range(T):
                _, past = model.classify_step(x[:, t], past)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for t in range(10):
                _, past = model.classify_step(x[:, t], past)
            torch.cuda.synchronize()
            res["ms_per_streamed_segment_bf16"] = round((time.perf_counter() - t0) * 1e3 / 10, 2)
            graph_step = model.capture_stream(past, x[:, 0])
            for t in range(3):
                graph_step(x[:, t])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for t in range(10):
                graph_step(x[:, t])
            torch.cuda.synchronize()
            res["ms_per_streamed_segment_graph_replay_bf16"] = round((time.perf_counter() - t0) * 1e3 / 10, 2)
            del past, graph_step
        del model
        torch.cuda.empty_cache()
    res["logits_bf16"] = [round(v, 5) for v in logits[False].flatten().tolist()]
    res["fp8_vs_bf16_logit_max_abs_diff"] = round((logits[True] - logits[False]).abs().max().item(), 6)
    return res
