"""Parity of the HIP backward (mvpa_backward through the FlashMVPA autograd function) with
reverse-mode differentiation of the oracle's closed-form MVPA in float64.

The oracle forward is pinned in tests/test_oracle.py; its gradient is what torch.autograd derives
from it (and tests/test_oracle.py::test_direct_gradcheck checks that derivation against finite
differences).  Tolerances: fp32 inputs max-abs <= 2e-5 + 1e-4 * max|ref| per gradient; bf16
inputs rel-L2 <= 2e-2 per gradient (inputs rounded to bf16 on both sides, gradients returned in
bf16)."""
import math
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "multi-variate-parallel-transformer_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

from oracle import mvpa_oracle as O  # noqa: E402
from mvpa_hip.synthetic import make_mvpa_inputs  # noqa: E402

pytestmark = pytest.mark.gpu

NAMES = ("q", "u", "vb", "z", "k", "k_time", "k_chan", "v")


def _oracle_grads(inp, d_out, window, chan_valid=None, time_bias=True, chan_bias=True):
    leaves = {n: getattr(inp, n).double().clone().requires_grad_(True) for n in NAMES}
    k_time = leaves["k_time"] if time_bias else leaves["k_time"] * 0
    k_chan = leaves["k_chan"] if chan_bias else leaves["k_chan"] * 0
    vb = leaves["vb"] if time_bias else leaves["vb"] * 0
    z = leaves["z"] if chan_bias else leaves["z"] * 0
    out = O.mvpa_direct(leaves["q"], leaves["k"], leaves["v"], leaves["u"], vb, z, k_time, k_chan,
                        window=window, chan_valid=chan_valid)
    grads = torch.autograd.grad((out * d_out.double()).sum(), [leaves[n] for n in NAMES],
                                allow_unused=True)
    return out.detach(), {n: (g if g is not None else torch.zeros_like(leaves[n])) for n, g in zip(NAMES, grads)}


def _gpu_grads(inp, d_out, window, dtype, chan_valid=None, time_bias=True, chan_bias=True):
    from attentions import flashmvpa
    hkv, dh = inp.u.shape
    t_len, c_len = inp.k_time.shape[1], inp.k_chan.shape[1]
    leaves = {n: getattr(inp, n).to(dtype).cuda().requires_grad_(True) for n in NAMES}
    out = flashmvpa(leaves["q"], leaves["u"].view(1, hkv, 1, dh), leaves["vb"].view(1, hkv, 1, dh),
                    leaves["z"].view(1, hkv, 1, dh), leaves["k"],
                    leaves["k_time"].view(1, hkv, t_len, dh), leaves["k_chan"].view(1, hkv, c_len, dh),
                    leaves["v"], True, 1.0 / math.sqrt(dh), window_size=window,
                    rel_bias_time=time_bias, rel_bias_chan=chan_bias,
                    chan_valid=chan_valid.cuda() if chan_valid is not None else None)
    out.backward(d_out.to(dtype).cuda())
    return out.detach().float().cpu(), {n: (leaves[n].grad.float().cpu() if leaves[n].grad is not None
                                            else torch.zeros_like(getattr(inp, n))) for n in NAMES}


CASES = [
    dict(B=2, C=8, T=32, H=4, Hkv=4, Dh=32, window=10),     # the reference's CPU-runnable size
    dict(B=1, C=3, T=13, H=4, Hkv=2, Dh=16, window=10),     # GQA, window active
    dict(B=2, C=5, T=7, H=2, Hkv=1, Dh=64, window=10),      # window vacuous, ragged C
    dict(B=1, C=4, T=14, H=2, Hkv=2, Dh=32, window=3),      # narrow window
    dict(B=1, C=6, T=9, H=2, Hkv=2, Dh=128, window=0),      # content everywhere
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{B}C{C}T{T}H{H}g{Hkv}D{Dh}w{window}".format(**c))
def test_backward_fp32_matches_oracle_autograd(case):
    cfg = dict(case)
    window = cfg.pop("window")
    inp = make_mvpa_inputs(seed=3, qkv_unit=True, **cfg)
    g = torch.Generator().manual_seed(11)
    d_out = torch.randn(inp.q.shape, generator=g)
    ref_out, ref = _oracle_grads(inp, d_out, window)
    out, got = _gpu_grads(inp, d_out, window, torch.float32)
    assert (out.double() - ref_out).abs().max().item() <= 1e-5
    for n in NAMES:
        err = (got[n].double() - ref[n]).abs().max().item()
        assert err <= 2e-5 + 1e-4 * ref[n].abs().max().item(), (n, err)


def test_backward_with_channel_validity():
    inp = make_mvpa_inputs(B=2, C=6, T=12, H=2, Hkv=2, Dh=32, seed=5, qkv_unit=True)
    valid = torch.tensor([[1, 1, 0, 1, 1, 0], [0, 1, 1, 1, 1, 1]], dtype=torch.bool)
    d_out = torch.randn(inp.q.shape, generator=torch.Generator().manual_seed(2))
    _, ref = _oracle_grads(inp, d_out, 10, chan_valid=valid)
    _, got = _gpu_grads(inp, d_out, 10, torch.float32, chan_valid=valid)
    for n in NAMES:
        err = (got[n].double() - ref[n]).abs().max().item()
        assert err <= 2e-5 + 1e-4 * ref[n].abs().max().item(), (n, err)
    # keys of absent channels receive no gradient at all
    absent = (~valid)[:, None, None, :].expand(2, 2, 12, 6).reshape(2, 2, 72)
    assert got["k"][absent].abs().max().item() == 0.0
    assert got["v"][absent].abs().max().item() == 0.0


def test_backward_bf16_within_tolerance():
    inp = make_mvpa_inputs(B=1, C=16, T=24, H=4, Hkv=2, Dh=64, seed=9, qkv_unit=True).round_to(torch.bfloat16)
    d_out = torch.randn(inp.q.shape, generator=torch.Generator().manual_seed(4)).bfloat16().float()
    _, ref = _oracle_grads(inp, d_out, 10)
    _, got = _gpu_grads(inp, d_out, 10, torch.bfloat16)
    for n in NAMES:
        rel = (got[n].double() - ref[n]).norm().item() / max(ref[n].norm().item(), 1e-30)
        assert rel <= 2e-2, (n, rel)


BF16_CASES = [
    dict(B=1, C=64, T=12, H=2, Hkv=2, Dh=64, window=10),      # two waves per time step
    dict(B=1, C=40, T=37, H=2, Hkv=1, Dh=64, window=10),      # ragged channels, two 32-step slabs, GQA
    dict(B=2, C=8, T=70, H=1, Hkv=1, Dh=64, window=4),        # three slabs, narrow window
    dict(B=1, C=33, T=9, H=2, Hkv=2, Dh=64, window=0),        # content everywhere; odd C (workspace rows padded to 36)
    dict(B=1, C=117, T=9, H=2, Hkv=1, Dh=64, window=2),       # two channel parts (64 + 53), four launches per pass, GQA
    dict(B=1, C=128, T=6, H=1, Hkv=1, Dh=64, window=10),      # two full channel parts
    dict(B=2, C=65, T=35, H=2, Hkv=2, Dh=64, window=3),       # second part of one channel; two slabs
    dict(B=1, C=36, T=9, H=2, Hkv=2, Dh=64, window=0),        # content everywhere, ragged second channel tile
    dict(B=1, C=32, T=21, H=2, Hkv=1, Dh=64, window=3),       # one channel tile, four key steps per workgroup, GQA
    dict(B=2, C=20, T=40, H=2, Hkv=2, Dh=64, window=5),       # one ragged channel tile, two slabs
    dict(B=1, C=64, T=45, H=1, Hkv=1, Dh=64, window=2),       # odd T: the last key pair of a workgroup is half empty
    # head dim 128: rows of 256 bytes in the LDS tiles, the key pass in quarters of 32 x 32 channels
    dict(B=1, C=32, T=21, H=2, Hkv=1, Dh=128, window=3),      # one channel tile, GQA
    dict(B=2, C=20, T=40, H=2, Hkv=2, Dh=128, window=5),      # one ragged channel tile, two slabs
    dict(B=1, C=64, T=12, H=2, Hkv=2, Dh=128, window=10),     # two channel tiles per query step, four key-pass launches
    dict(B=1, C=40, T=37, H=2, Hkv=1, Dh=128, window=10),     # ragged second tile, two slabs, GQA
    dict(B=1, C=117, T=9, H=2, Hkv=1, Dh=128, window=2),      # two channel parts: 4 query-pass, 16 key-pass launches
    dict(B=1, C=128, T=6, H=1, Hkv=1, Dh=128, window=10),     # two full channel parts
    dict(B=2, C=65, T=35, H=2, Hkv=2, Dh=128, window=3),      # second part of one channel; two slabs
    dict(B=1, C=33, T=9, H=2, Hkv=2, Dh=128, window=0),       # content everywhere; odd C
]


@pytest.mark.parametrize("case", BF16_CASES, ids=lambda c: "B{B}C{C}T{T}H{H}g{Hkv}D{Dh}w{window}".format(**c))
def test_backward_bf16_mfma_query_pass(case):
    """bf16, Dh = 64 or 128, C <= 128 takes the MFMA passes (dq, dk, dv, bias-table gradients)."""
    cfg = dict(case)
    window = cfg.pop("window")
    inp = make_mvpa_inputs(seed=13, qkv_unit=True, **cfg).round_to(torch.bfloat16)
    d_out = torch.randn(inp.q.shape, generator=torch.Generator().manual_seed(6)).bfloat16().float()
    valid = None
    if cfg["C"] in (40, 20, 117):
        valid = torch.ones(cfg["B"], cfg["C"], dtype=torch.bool)
        valid[:, [3, 17, cfg["C"] - 1]] = False
    _, ref = _oracle_grads(inp, d_out, window, chan_valid=valid)
    _, got = _gpu_grads(inp, d_out, window, torch.bfloat16, chan_valid=valid)
    for n in NAMES:
        rel = (got[n].double() - ref[n]).norm().item() / max(ref[n].norm().item(), 1e-30)
        assert rel <= 2e-2, (n, rel)


def test_backward_rows_are_causal():
    """do confined to the first time steps must leave dk/dv of later keys exactly zero."""
    inp = make_mvpa_inputs(B=1, C=4, T=10, H=2, Hkv=2, Dh=32, seed=1, qkv_unit=True)
    d_out = torch.zeros(inp.q.shape)
    d_out[:, :, : 3 * 4] = torch.randn(1, 2, 12, 32, generator=torch.Generator().manual_seed(8))
    _, got = _gpu_grads(inp, d_out, 10, torch.float32)
    assert got["k"][:, :, 3 * 4:].abs().max().item() == 0.0
    assert got["v"][:, :, 3 * 4:].abs().max().item() == 0.0
    assert got["q"][:, :, 3 * 4:].abs().max().item() == 0.0


@pytest.mark.parametrize("flags", [dict(time_bias=False), dict(chan_bias=False)],
                         ids=lambda f: "+".join(sorted(f)))
def test_backward_bf16_mfma_bias_flags(flags):
    """The matrix-core passes with a bias term switched off: its parameters get zero gradient."""
    inp = make_mvpa_inputs(B=1, C=64, T=20, H=2, Hkv=2, Dh=64, seed=21, qkv_unit=True).round_to(torch.bfloat16)
    d_out = torch.randn(inp.q.shape, generator=torch.Generator().manual_seed(3)).bfloat16().float()
    _, ref = _oracle_grads(inp, d_out, 4, **flags)
    _, got = _gpu_grads(inp, d_out, 4, torch.bfloat16, **flags)
    for n in NAMES:
        if ref[n].abs().max().item() == 0.0:
            assert got[n].abs().max().item() == 0.0, n
            continue
        rel = (got[n].double() - ref[n]).norm().item() / max(ref[n].norm().item(), 1e-30)
        assert rel <= 2e-2, (n, rel)


def test_backward_bf16_mfma_rows_are_causal():
    """As test_backward_rows_are_causal, on the matrix-core passes."""
    inp = make_mvpa_inputs(B=1, C=32, T=10, H=2, Hkv=2, Dh=64, seed=1, qkv_unit=True)
    d_out = torch.zeros(inp.q.shape)
    d_out[:, :, : 3 * 32] = torch.randn(1, 2, 96, 64, generator=torch.Generator().manual_seed(8))
    _, got = _gpu_grads(inp, d_out, 10, torch.bfloat16)
    assert got["k"][:, :, 3 * 32:].abs().max().item() == 0.0
    assert got["v"][:, :, 3 * 32:].abs().max().item() == 0.0
    assert got["q"][:, :, 3 * 32:].abs().max().item() == 0.0


@pytest.mark.parametrize("cfg", [dict(B=4, C=64, T=128, H=16, Hkv=16, Dh=64),
                                 dict(B=1, C=128, T=128, H=4, Hkv=2, Dh=128)],
                         ids=["c2", "C128-Dh128-GQA"])
def test_backward_bf16_full_size_invariants(cfg):
    """At the benchmark shape (B4 C64 T128 H16 Dh64, too large for the float64 oracle) and at the
    base model's channels, head dim and head grouping (C128 Dh128, two query heads per kv head) the
    gradients must satisfy what the softmax fixes for ANY d_o:
      * dS rows sum to zero, so every row of dbias_time and of dbias_chan sums to zero
        (up to the bf16 rounding of the probabilities: <= 1e-2 of the absolute sum of the row of
        dbias_chan, which stands for sum_keys |dS|);
      * with d_o = 1 the columns of dv are the column sums of P, so dv summed over the keys of a
        (batch, kv head) equals the number of queries of the group's heads, N * H/Hkv."""
    import mvpa_hip
    inp = make_mvpa_inputs(seed=0, **cfg).to("cuda", torch.bfloat16)
    out, lse = mvpa_hip.mvpa_forward(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                                     return_lse=True)
    d_o = torch.randn(out.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(5)).bfloat16()
    dq, dk, dv, dbt, dbc = mvpa_hip.mvpa_backward(inp.q, inp.k, inp.v, out, d_o, lse, inp.u, inp.vb, inp.z,
                                                  inp.k_time, inp.k_chan)
    for t in (dq, dk, dv, dbt, dbc):
        assert torch.isfinite(t).all()
    scale = dbc.abs().sum(-1)                          # ~ sum_keys |dS| of the row (measured: ratio <= 3.4e-3)
    for g in (dbt, dbc):
        rows = g.sum(-1).abs()
        assert (rows <= 1e-2 * scale).all(), (rows / scale).max().item()
    # the two tables hold the same dS, summed differently
    assert torch.allclose(dbt.sum(-1), dbc.sum(-1), atol=1e-4, rtol=0)
    ones = torch.ones_like(out)
    _, _, dv1, _, _ = mvpa_hip.mvpa_backward(inp.q, inp.k, inp.v, out, ones, lse, inp.u, inp.vb, inp.z,
                                             inp.k_time, inp.k_chan)
    n_q = cfg["T"] * cfg["C"] * (cfg["H"] // cfg["Hkv"])
    tot = dv1.sum(2)                                  # [B,Hkv,Dh]
    assert (tot / n_q - 1).abs().max().item() <= 2e-3, (tot / n_q - 1).abs().max().item()


def test_backward_bf16_strided_inputs_match_contiguous():
    """q, k, v, o, d_o as head-interleaved views ([B,N,H,Dh] buffers, the layout the layer's fused
    projection produces): the same gradients, bit for bit, as from contiguous copies."""
    import mvpa_hip
    cfg = dict(B=2, C=48, T=20, H=4, Hkv=2, Dh=64)
    inp = make_mvpa_inputs(seed=4, qkv_unit=True, **cfg).to("cuda", torch.bfloat16)
    tabs = (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)
    out, lse = mvpa_hip.mvpa_forward(inp.q, inp.k, inp.v, *tabs, return_lse=True)
    d_o = torch.randn(out.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(1)).bfloat16()
    ref = mvpa_hip.mvpa_backward(inp.q, inp.k, inp.v, out, d_o, lse, *tabs)

    def interleave(t):                      # [B,h,N,Dh] -> view of a [B,N,h,Dh] buffer
        return t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    q, k, v, o, g = (interleave(t) for t in (inp.q, inp.k, inp.v, out, d_o))
    assert not q.is_contiguous() and q.stride(-1) == 1
    got = mvpa_hip.mvpa_backward(q, k, v, o, g, lse, *tabs)
    for a, b in zip(got, ref):
        assert torch.equal(a, b)
