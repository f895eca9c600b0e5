"""Differential sweep on the GPU: the bf16 and fp16 matrix-core kernels (forward, both backward passes)
against the fp32 kernels of the same library, on seeded random shapes the oracle would take too
long for (ragged channel counts up to 128, odd time lengths, GQA, narrow / vacuous / zero windows, absent
channels).  The fp32 kernels are themselves pinned against the oracle in test_mvpa_gpu.py and
test_backward_gpu.py.  Tolerances: forward max-abs <= 2e-2 (as for bf16 against the oracle),
every gradient rel-L2 <= 2e-2; rows of absent channels are excluded (any finite value is valid
there)."""
import os
import random
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "multi-variate-parallel-transformer_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

from mvpa_hip.synthetic import make_mvpa_inputs  # noqa: E402

pytestmark = pytest.mark.gpu


def _compare_backward(d16, d32, o16, l16, o32, l32, live, seed, kw):
    """Both backward passes on the matrix cores against the fp32 pair: every gradient rel-L2 <= 2e-2."""
    import mvpa_hip
    tabs16 = (d16.u, d16.vb, d16.z, d16.k_time, d16.k_chan)
    tabs32 = (d32.u, d32.vb, d32.z, d32.k_time, d32.k_chan)
    d_o = torch.randn(o32.shape, device="cuda",
                      generator=torch.Generator("cuda").manual_seed(seed)).bfloat16()
    g16 = mvpa_hip.mvpa_backward(d16.q, d16.k, d16.v, o16, d_o, l16, *tabs16, **kw)
    g32 = mvpa_hip.mvpa_backward(d32.q, d32.k, d32.v, o32, d_o.float(), l32, *tabs32, **kw)
    for name, a, b in zip(("dq", "dk", "dv", "dbias_time", "dbias_chan"), g16, g32):
        if name in ("dq", "dbias_time", "dbias_chan"):       # per-query outputs
            a, b = a * live, b * live
        assert torch.isfinite(a).all(), name
        ref_norm = b.norm()
        if name == "dbias_time":
            # both tables sum the same dS; with few time steps the rows of this one approach the
            # row sums of dS, which are zero up to rounding (exactly so at T = 1): measure its
            # error against the larger of the two tables
            ref_norm = torch.maximum(ref_norm, (g32[4] * live).norm())
        rel = ((a - b).norm() / ref_norm.clamp_min(1e-20)).item()
        assert rel <= 2e-2, (name, rel)


def _cases(n=24, seed=20240):
    rng = random.Random(seed)
    out = []
    for it in range(n):
        hkv, grp = rng.choice([1, 2, 4]), rng.choice([1, 2, 3])
        out.append(dict(
            B=rng.choice([1, 2, 3]), C=rng.choice([4, 8, 12, 20, 32, 33, 36, 48, 60, 64, 65, 72, 100, 117, 128]),
            T=rng.choice([1, 2, 3, 5, 8, 13, 16, 31, 32, 33, 47, 64, 65, 96]),
            H=hkv * grp, Hkv=hkv, window=rng.choice([0, 1, 2, 5, 10, 200]),
            absent=rng.random() < 0.4, seed=it))
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: "B{B}C{C}T{T}H{H}g{Hkv}w{window}{a}".format(
    a="v" if c["absent"] else "", **c))
def test_mfma_paths_match_fp32_kernels(case):
    import mvpa_hip
    B, C, T, H, Hkv = (case[k] for k in ("B", "C", "T", "H", "Hkv"))
    inp = make_mvpa_inputs(B=B, C=C, T=T, H=H, Hkv=Hkv, Dh=64, seed=case["seed"],
                           qkv_unit=True).round_to(torch.bfloat16)
    valid = None
    if case["absent"] and C > 2:
        rng = random.Random(case["seed"])
        valid = torch.ones(B, C, dtype=torch.bool)
        for b in range(B):
            valid[b, rng.sample(range(C), k=max(1, C // 5))] = False
        valid = valid.cuda()
    d16, d32 = inp.to("cuda", torch.bfloat16), inp.to("cuda", torch.float32)
    kw = dict(window=case["window"], chan_valid=valid)
    tabs16 = (d16.u, d16.vb, d16.z, d16.k_time, d16.k_chan)
    tabs32 = (d32.u, d32.vb, d32.z, d32.k_time, d32.k_chan)
    o16, l16 = mvpa_hip.mvpa_forward(d16.q, d16.k, d16.v, *tabs16, return_lse=True,
                                     kernel=mvpa_hip.KERNEL_MFMA, **kw)
    o32, l32 = mvpa_hip.mvpa_forward(d32.q, d32.k, d32.v, *tabs32, return_lse=True, **kw)
    live = torch.ones(B, 1, T, C, dtype=torch.bool, device="cuda") if valid is None \
        else valid[:, None, None, :].expand(B, 1, T, C)
    live = live.reshape(B, 1, T * C, 1)
    assert ((o16.float() - o32) * live).abs().max().item() <= 2e-2
    assert ((l16 - l32) * live[..., 0]).abs().max().item() <= 2e-2
    if 32 < C <= 128:         # the build in which a wave owns 32 queries x 64 columns (here: a workgroup on 2 or 4 time steps)
        o16w, l16w = mvpa_hip.mvpa_forward(d16.q, d16.k, d16.v, *tabs16, return_lse=True,
                                           kernel=mvpa_hip.KERNEL_MFMA_SPLIT, **kw)
        assert ((o16w.float() - o32) * live).abs().max().item() <= 2e-2
        assert ((l16w - l32) * live[..., 0]).abs().max().item() <= 2e-2
    if 32 < C <= 64:          # the build in which a wave owns a whole time step, at every length
        o16s, l16s = mvpa_hip.mvpa_forward(d16.q, d16.k, d16.v, *tabs16, return_lse=True,
                                           kernel=mvpa_hip.KERNEL_MFMA_STEP, **kw)
        assert ((o16s.float() - o32) * live).abs().max().item() <= 2e-2
        assert ((l16s - l32) * live[..., 0]).abs().max().item() <= 2e-2
    _compare_backward(d16, d32, o16, l16, o32, l32, live, case["seed"], kw)


def _forward_cases(n=20, seed=777):
    rng = random.Random(seed)
    out = []
    for it in range(n):
        hkv, grp = rng.choice([1, 2]), rng.choice([1, 2, 3])
        out.append(dict(
            B=rng.choice([1, 2]), Dh=rng.choice([32, 128]),
            C=rng.choice([8, 20, 32, 33, 48, 64, 65, 80, 100, 117, 128]),
            T=rng.choice([2, 12, 13, 24, 33, 47, 64, 70]),
            H=hkv * grp, Hkv=hkv, window=rng.choice([0, 2, 10, 10, 10]),
            absent=rng.random() < 0.4, seed=1000 + it))
    return out


@pytest.mark.parametrize("case", _forward_cases(), ids=lambda c: "D{Dh}B{B}C{C}T{T}H{H}g{Hkv}w{window}{a}".format(
    a="v" if c["absent"] else "", **c))
def test_mfma_forward_matches_fp32_kernel_at_other_head_sizes(case):
    """Head sizes 32 and 128 (every build of the matrix-core forward the dispatcher can pick for
    them, far steps included) against the fp32 kernel: output max-abs <= 2e-2, log-sum-exp 2e-2.
    The same inputs as fp16 tensors (bf16 values are fp16 values here) on the fp16 matrix-core
    kernel: max-abs <= 1e-3, log-sum-exp 2e-3.  At head size 128 also both backward passes on the
    matrix cores against the fp32 pair."""
    import mvpa_hip
    B, C, T, H, Hkv, Dh = (case[k] for k in ("B", "C", "T", "H", "Hkv", "Dh"))
    inp = make_mvpa_inputs(B=B, C=C, T=T, H=H, Hkv=Hkv, Dh=Dh, seed=case["seed"],
                           qkv_unit=True, table_std=0.2).round_to(torch.bfloat16)
    valid = None
    if case["absent"]:
        rng = random.Random(case["seed"])
        valid = torch.ones(B, C, dtype=torch.bool)
        for b in range(B):
            valid[b, rng.sample(range(C), k=max(1, C // 5))] = False
        valid = valid.cuda()
    d16, d32 = inp.to("cuda", torch.bfloat16), inp.to("cuda", torch.float32)
    kw = dict(window=case["window"], chan_valid=valid, return_lse=True)
    o16, l16 = mvpa_hip.mvpa_forward(d16.q, d16.k, d16.v, d16.u, d16.vb, d16.z, d16.k_time, d16.k_chan,
                                     kernel=mvpa_hip.KERNEL_MFMA, **kw)
    o32, l32 = mvpa_hip.mvpa_forward(d32.q, d32.k, d32.v, d32.u, d32.vb, d32.z, d32.k_time, d32.k_chan, **kw)
    live = torch.ones(B, 1, T, C, dtype=torch.bool, device="cuda") if valid is None \
        else valid[:, None, None, :].expand(B, 1, T, C)
    live = live.reshape(B, 1, T * C, 1)
    assert torch.isfinite(o16.float()).all()
    assert ((o16.float() - o32) * live).abs().max().item() <= 2e-2
    assert ((l16 - l32) * live[..., 0]).abs().max().item() <= 2e-2
    if Dh == 128 and 32 < C <= 128:      # the build with the output columns split over two waves
        o16s, l16s = mvpa_hip.mvpa_forward(d16.q, d16.k, d16.v, d16.u, d16.vb, d16.z, d16.k_time, d16.k_chan,
                                           kernel=mvpa_hip.KERNEL_MFMA_SPLIT, **kw)
        assert torch.isfinite(o16s.float()).all()
        assert ((o16s.float() - o32) * live).abs().max().item() <= 2e-2
        assert ((l16s - l32) * live[..., 0]).abs().max().item() <= 2e-2
    dh = inp.to("cuda", torch.float16)
    oh, lh = mvpa_hip.mvpa_forward(dh.q, dh.k, dh.v, dh.u, dh.vb, dh.z, dh.k_time, dh.k_chan,
                                   kernel=mvpa_hip.KERNEL_MFMA, **kw)
    assert oh.dtype == torch.float16 and torch.isfinite(oh.float()).all()
    assert ((oh.float() - o32) * live).abs().max().item() <= 1e-3
    assert ((lh - l32) * live[..., 0]).abs().max().item() <= 2e-3
    if Dh == 128:
        _compare_backward(d16, d32, o16, l16, o32, l32, live, case["seed"],
                          dict(window=case["window"], chan_valid=valid))
