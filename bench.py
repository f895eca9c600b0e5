#!/usr/bin/env python3
"""Benchmark of the MVPA forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4attn|c5attn] [--no-cpu]
                    [--no-model] [--no-stream] [--no-backward] [--no-extra] [--no-base-model]
                    [--base-stream] [--copy-probe] [--prewarm P]

A step is one fused MVPA forward (one kernel launch) over one batch of synthetic inputs that
are already resident in HBM.  The default workload is the configuration the headline metric
is quoted on: B=4, C=64, T=128, H=16, Dh=64, bf16, time-causal, window 10.  Prints ONE JSON
line with the metric, the roofline of the attention kernel (achieved = algorithmic flops per
launch / HIP-event time per launch) and a bounded CPU baseline (the oracle's op-by-op
restatement of the reference PyTorch path on this box's host cores).  Beside them, never part
of `value`: `backward` (one mvpa_backward call on the same workload), `mvpformer_s` (the
MVPFormer-S forward in windows per second, with the oracle stack on the host cores beside it),
`mvpformer_s_stream` (one new segment of a stream against cached keys and values, beside the
full forward over the same window), `mvpa_c3` and `mvpa_c5attn` (the irregular-channel
configuration and the base model's attention shape, a few launches each: time, algorithmic
TFLOP/s, fraction of the bf16 peak, kernel, and the time of one mvpa_backward call on the same
inputs) and `mvpformer_base` (the base-size classification
forward at B1 C128 T512, bf16 and fp8 QK^T, with the logit gap between the two).

The GPU's clocks take a few dozen milliseconds of work to reach their steady state after a
process starts.  Before the W warm-up steps the benchmark therefore runs a fixed number of
launches of the same kernel (`prewarm_launches` in the output, outside the timed region), so
that the figure does not depend on how small W is.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "multi-variate-parallel-transformer_amd")
for _p in (PKG, ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)

BF16_DENSE_PEAK_TFLOPS = 2500.0       # MI355X published dense bf16 MFMA peak

# HBM bytes per launch of the attention kernel from rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by
# what the same counters read for a plain device copy of known size; the profile summary named
# beside each figure holds the two counter runs.
MEASURED_TRAFFIC_BYTES = {"c2": (702.9e6, "profiles/mvpa_mfma64_kernel_c2.md"),
                          "c3": (4.68e9, "profiles/mvpa_mfma128_kernel_c3.md"),
                          "c5attn": (11.51e9, "profiles/mvpa_mfma128_kernel_c5attn.md")}
PREWARM_LAUNCHES = 150

WORKLOADS = {
    "c2": dict(B=4, C=64, T=128, H=16, Hkv=16, Dh=64, validity=False),
    "c3": dict(B=8, C=117, T=256, H=16, Hkv=16, Dh=64, validity=True),
    # the attention shape inside configuration c5 (the base model: one sample, 128 channels, 512 segments)
    "c5attn": dict(B=1, C=128, T=512, H=16, Hkv=8, Dh=128, validity=False),
    # the attention shape inside configuration c4 (MVPFormer-S: 64 channels, 64 segments, 3 heads per kv head)
    "c4attn": dict(B=4, C=64, T=64, H=12, Hkv=4, Dh=64, validity=False),
}


def _forward_kernel_name(cfg):
    """The build of the bf16 forward that the library's own choice (MVPA_KERNEL_AUTO) runs for a
    workload: the rule of mvpa_forward in csrc/mvpa_api.hip."""
    if (cfg["Dh"] in (64, 128) and 64 < cfg["C"] <= 128) or (cfg["Dh"] == 128 and 32 < cfg["C"] <= 64):
        return "mvpa::d128::mvpa_mfma128_kernel"
    if cfg["Dh"] == 64 and 32 < cfg["C"] <= 64 and cfg["T"] >= 128:
        return "mvpa::q64::mvpa_mfma64_kernel"
    return "mvpa::mvpa_mfma_kernel"


def algorithmic_flops(B, H, T, C, Dh, window=10):
    """Flops the operator needs: PV for every causally visible pair, QK^T only where the content
    term is kept (|tq-tk| <= window, plus the whole last time row), and the two bias-table
    contractions N*(T+C)."""
    n = T * C
    p_causal = C * C * T * (T + 1) // 2
    if window > 0 and T > window + 1:
        w1 = window + 1
        p_window = C * C * (w1 * (w1 + 1) // 2 - w1 + w1 * (T - w1) + T)
    else:
        p_window = p_causal
    return B * H * 2 * Dh * (p_causal + p_window + n * (T + C))


def _extra_workload(key, warmup=3, steps=5, backward=True):
    """One of the other benchmark shapes on the library's own kernel choice: HIP-event time per
    launch over `steps` launches, algorithmic TFLOP/s and the fraction of the dense bf16 peak;
    with `backward`, the time of one mvpa_backward call on the same inputs beside it."""
    import torch
    import mvpa_hip
    from mvpa_hip.synthetic import make_mvpa_inputs

    cfg = WORKLOADS[key]
    B, C, T, H, Hkv, Dh = (cfg[k] for k in ("B", "C", "T", "H", "Hkv", "Dh"))
    d = make_mvpa_inputs(B=B, C=C, T=T, H=H, Hkv=Hkv, Dh=Dh, seed=0, qkv_unit=True,
                         validity=cfg["validity"]).to("cuda:0", torch.bfloat16)
    out = torch.empty_like(d.q)

    def step():
        mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                              chan_valid=d.chan_valid, out=out)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / steps
    flops = algorithmic_flops(B, H, T, C, Dh)
    tf = flops / (ms * 1e-3) / 1e12
    res = {"workload": f"B={B} C={C} T={T} H={H} Hkv={Hkv} Dh={Dh}"
                       + (", per-sample channel validity" if cfg["validity"] else ""),
           "ms": round(ms, 4), "steps": steps, "tflops": round(tf, 1),
           "frac": round(tf / BF16_DENSE_PEAK_TFLOPS, 4), "algorithmic_flops": flops,
           "kernel": _forward_kernel_name(cfg)}
    if backward:
        _, lse = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                       chan_valid=d.chan_valid, return_lse=True)
        d_o = torch.randn_like(out)

        def bwd():
            return mvpa_hip.mvpa_backward(d.q, d.k, d.v, out, d_o, lse, d.u, d.vb, d.z, d.k_time,
                                          d.k_chan, chan_valid=d.chan_valid)
        bwd()
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(2):
            bwd()
        ev1.record()
        torch.cuda.synchronize()
        res["backward_ms"] = round(ev0.elapsed_time(ev1) / 2, 3)
    return res


def cpu_baseline(cfg, budget_s=8.0):
    """Oracle restatement of the reference PyTorch MVPA (same op sequence, same N^2 traffic) on
    the host CPU for a bounded sample: whole (b, h) slices of the workload, fp32."""
    import torch
    from mvpa_hip.synthetic import make_mvpa_inputs
    from oracle import mvpa_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    T, C, Dh = cfg["T"], cfg["C"], cfg["Dh"]
    # one (b, h) slice at a time; c3 is cut to a prefix of its time steps to bound memory
    Ts = min(T, 128)
    inp = make_mvpa_inputs(B=1, C=C, T=Ts, H=1, Dh=Dh, seed=1, qkv_unit=True)
    q = inp.q.view(1, 1, Ts, C, Dh)
    k = inp.k.view(1, 1, Ts, C, Dh)
    v = inp.v.view(1, 1, Ts, C, Dh)
    tk = inp.k_time.view(1, 1, Ts, 1, Dh)
    ck = inp.k_chan.view(1, 1, 1, C, Dh)
    bias = torch.cat([inp.u.reshape(-1), inp.vb.reshape(-1), inp.z.reshape(-1)])
    flops = algorithmic_flops(1, 1, Ts, C, Dh)
    with torch.no_grad():
        O.rel_attn(q, k, tk, ck, v, bias)                      # warm-up
        reps, t0 = 0, time.perf_counter()
        while True:
            O.rel_attn(q, k, tk, ck, v, bias)
            reps += 1
            el = time.perf_counter() - t0
            if el >= budget_s or reps >= 20:
                break
    per = el / reps
    return {
        "value": round(flops / per / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{reps} x one (b,h) slice of the workload (T={Ts}, C={C}, Dh={Dh}, fp32), "
                  f"{per * 1e3:.0f} ms each; algorithmic flops as for the GPU line",
    }


def cpu_baseline_model(B=1, C=64, T=64, seg=512):
    """The oracle stack (encoder, parallel blocks with the op-by-op attention restatement, final
    norm) on the host cores, fp32, with MVPFormer-S dims: one window at full length with one and
    with two blocks; a block's cost is the difference, and the 12-block figure is extrapolated
    from it (stated in the result)."""
    import torch
    from mvpa_hip.synthetic import make_ieeg
    from models.configs import MVPFORMER_S
    from oracle import mvpa_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    E, H, Hkv, inner = (MVPFORMER_S[k] for k in ("n_embd", "n_head", "n_head_kv", "n_inner"))
    kv = E // H * Hkv
    g = torch.Generator().manual_seed(0)
    rn = lambda *shape: torch.randn(*shape, generator=g) * 0.02      # noqa: E731
    dwt = sum(O.dwt_sizes(seg))
    params = {"encoder.ln.weight": torch.ones(dwt), "encoder.proj.weight": rn(E, dwt),
              "mvpformer.ln_f.weight": torch.ones(E),
              "mvpformer.positional_embedding.weight": rn(T, E),
              "mvpformer.channel_embedding.weight": rn(C, E)}
    for i in range(1):
        pre = f"mvpformer.h.{i}."
        params.update({pre + "ln_1.weight": torch.ones(E), pre + "attn.q_attn.weight": rn(E, E),
                       pre + "attn.c_attn.weight": rn(2 * kv, E), pre + "attn.position_net.weight": rn(kv, E),
                       pre + "attn.channel_net.weight": rn(kv, E), pre + "attn.c_proj.weight": rn(E, E),
                       pre + "attn.attn_bias": rn(3 * kv), pre + "mlp.gate_proj.weight": rn(inner, E),
                       pre + "mlp.up_proj.weight": rn(inner, E), pre + "mlp.down_proj.weight": rn(E, inner)})
    x = make_ieeg(B, C, T, seg, seed=0)
    times = {}
    with torch.no_grad():
        O.mvpformer_forward(x[:, :8], params, dict(n_layer=1, n_head=H, n_head_kv=Hkv))   # thread pool warm-up
        for n_layer in (0, 1):
            for _ in range(2):      # the second call is the one reported: the first also pays for
                t0 = time.perf_counter()         # allocator and thread-pool warm-up at this size
                O.mvpformer_forward(x, params, dict(n_layer=n_layer, n_head=H, n_head_kv=Hkv))
                times[n_layer] = time.perf_counter() - t0
    per_block = max(times[1] - times[0], 1e-9)
    full = times[0] + MVPFORMER_S["n_layer"] * per_block
    return {"value": round(B / full, 4), "unit": "windows/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"oracle stack, fp32, B={B} C={C} T={T} segments of {seg} samples: encoder + final "
                      f"norm {times[0]:.2f} s, one block {per_block:.2f} s (each timed twice, the second "
                      f"call reported); extrapolated to 12 blocks: {full:.1f} s per window"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--prewarm", type=int, default=PREWARM_LAUNCHES,
                    help="launches before the warm-up steps that bring the clocks up (untimed)")
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-model", action="store_true", help="skip the MVPFormer-S forward leg")
    ap.add_argument("--no-stream", action="store_true", help="skip the MVPFormer-S streamed-segment leg")
    ap.add_argument("--no-backward", action="store_true", help="skip the MVPA backward leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the c3 and c5-attention legs")
    ap.add_argument("--no-base-model", action="store_true",
                    help="skip the base-size classification forward (B1 C128 T512, bf16 and fp8 QK^T)")
    ap.add_argument("--base-model", action="store_true", help=argparse.SUPPRESS)   # (now the default)
    ap.add_argument("--base-stream", action="store_true",
                    help="with the base-size forward: also time its streamed segments")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 256 MiB device copy (calibrates HBM traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures ONE GPU (the MVPA forward shards over batch and "
              "heads with no exchange step); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import mvpa_hip
    from mvpa_hip.synthetic import make_mvpa_inputs

    mvpa_hip.load_library()           # fails loudly if the HIP extension is missing
    cfg = WORKLOADS[args.workload]
    B, C, T, H, Hkv, Dh = (cfg[k] for k in ("B", "C", "T", "H", "Hkv", "Dh"))
    inp = make_mvpa_inputs(B=B, C=C, T=T, H=H, Hkv=Hkv, Dh=Dh, seed=0, qkv_unit=True,
                           validity=cfg["validity"])
    d = inp.to("cuda:0", torch.bfloat16)
    torch.cuda.set_device(0)
    out = torch.empty_like(d.q)

    def step():
        mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                              chan_valid=d.chan_valid, out=out)

    if args.copy_probe:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(max(0, args.prewarm)):
        step()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()                      # kernels go to torch's current stream, so these events see them
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps
    flops = algorithmic_flops(B, H, T, C, Dh)
    tflops = flops / (wall_ms * 1e-3) / 1e12
    kern_tflops = flops / (kern_ms * 1e-3) / 1e12

    line = {
        "metric": "MVPA fwd TFLOP/s (algorithmic flops), bf16, 1 GPU",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "prewarm_launches": max(0, args.prewarm),
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: MVPA forward B={B} C={C} T={T} H={H} Hkv={Hkv} "
                               f"Dh={Dh}, window 10, time-causal"
                               + (", per-sample channel validity" if cfg["validity"] else ""),
                   "algorithmic_flops": flops},
        "roofline": {"bound": "mfma", "achieved": round(kern_tflops, 2),
                     "peak": BF16_DENSE_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(kern_tflops / BF16_DENSE_PEAK_TFLOPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload, (None, None))[0],
                     "traffic_source": MEASURED_TRAFFIC_BYTES.get(args.workload, (None, None))[1],
                     "kernel": _forward_kernel_name(cfg), "kernel_ms": round(kern_ms, 4)},
    }
    if not args.no_backward and C <= 128:   # shapes the matrix-core backward serves
        # the backward of the same workload (reported beside the headline, never part of `value`):
        # both passes of mvpa_backward, gradients and workspace allocated outside the timed region
        # by torch's caching allocator after the first call
        _, lse = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                       chan_valid=d.chan_valid, return_lse=True)
        d_o = torch.randn_like(out)

        def bwd():
            return mvpa_hip.mvpa_backward(d.q, d.k, d.v, out, d_o, lse, d.u, d.vb, d.z, d.k_time,
                                          d.k_chan, chan_valid=d.chan_valid)
        n_bwd = max(1, min(args.steps, 20))
        for _ in range(max(1, min(args.warmup, 5))):
            bwd()
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(n_bwd):
            bwd()
        ev1.record()
        torch.cuda.synchronize()
        line["backward"] = {"ms_per_step": round(ev0.elapsed_time(ev1) / n_bwd, 4), "steps": n_bwd,
                            "kernels": "mvpa_bwd_query_mfma_kernel + mvpa_bwd_key_mfma_kernel",
                            "outputs": "dq (content share), dk, dv, dbias_time, dbias_chan (fp32)"}
    if not args.no_extra:
        # the other attention shapes of the benchmark set, a few launches each, beside the headline
        # and never part of `value`: the irregular-channel configuration and the attention shape of
        # the base model
        for key in ("c3", "c5attn"):
            if key != args.workload:
                line["mvpa_" + key] = _extra_workload(key, backward=not args.no_backward)
    if not args.no_model:
        try:
            from bench_model import mvpformer_s_windows_per_s
            line["mvpformer_s"] = mvpformer_s_windows_per_s()
            if not args.no_stream:
                from bench_model import mvpformer_s_stream_step_ms
                line["mvpformer_s_stream"] = mvpformer_s_stream_step_ms()
        except ImportError:
            line["mvpformer_s"] = None
    if not args.no_base_model:
        from bench_model import mvpformer_base_forward_ms
        line["mvpformer_base"] = mvpformer_base_forward_ms(stream=args.base_stream)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(cfg)
        if line.get("mvpformer_s"):
            line["mvpformer_s"]["cpu_baseline"] = cpu_baseline_model()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
