"""GPU parity of the fused MVPA forward (through the C ABI) against the CPU oracle."""
import math

import pytest
import torch

import mvpa_hip
from mvpa_hip.synthetic import make_mvpa_inputs
from oracle import mvpa_oracle as O

pytestmark = pytest.mark.gpu

F32_MAX_ABS = 1e-5            # fp32 kernel vs fp32/fp64 oracle
BF16_MAX_ABS = 2e-2           # bf16 kernel vs oracle on the same bf16-rounded inputs
BF16_REL_L2 = 5e-3


def _oracle(inp, dtype=torch.float64, **kw):
    return O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                         chan_valid=inp.chan_valid, dtype=dtype, **kw)


def _gpu(inp, dtype, **kw):
    d = inp.to("cuda", dtype)
    return mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                 chan_valid=d.chan_valid, **kw)


def _rel_l2(a, b):
    return ((a - b).norm() / b.norm()).item()


def test_debug_maps_bit_exact():
    """Gather indices and masks as the kernels compute them == the reference's shift and mask
    construction, element for element (layers/mvpa.py:127-159, 230-264)."""
    T, C, W = 14, 5, 10
    N = T * C
    valid = torch.tensor([1, 0, 1, 1, 0], dtype=torch.bool)
    ti, ci, mb = mvpa_hip.debug_maps(T, C, W, chan_valid=valid.cuda())
    ti, ci, mb = ti.cpu(), ci.cpu(), mb.cpu()
    # the reference's shifts applied to iota-coded tables give the gathered column
    xt = torch.arange(T, dtype=torch.float32).expand(1, 1, N, T).contiguous()
    xc = torch.arange(C, dtype=torch.float32).expand(1, 1, N, C).contiguous()
    rt = O.repeat_channel(O.rel_shift(xt), C)[0, 0]
    rc = O.repeat_time(O.rel_shift_chan(xc), T)[0, 0]
    n = torch.arange(N)
    causal = (n // C)[None, :] <= (n // C)[:, None]
    assert torch.equal(ti[causal], rt[causal].to(torch.int32))
    assert (ti[~causal] == -1).all()
    assert torch.equal(ci, rc.to(torch.int32))
    ones = torch.ones((T, T), dtype=torch.bool)
    win = torch.tril(ones, diagonal=W) & torch.triu(ones, diagonal=-W)
    win = win.repeat_interleave(C, 0).repeat_interleave(C, 1)
    win[-C:] = True
    vis = causal & valid.repeat(T)[None, :]
    assert torch.equal(mb & 1, vis.to(torch.uint8))
    assert torch.equal((mb >> 1) & 1, win.to(torch.uint8))


def test_fp32_config1_parity():
    """Config c1 (B2 C8 T32 H4 Dh32, q/k/v ~ N(0,1), seed 0), fp32: max-abs <= 1e-5 against
    both oracle statements and the committed golden output."""
    inp = make_mvpa_inputs(B=2, C=8, T=32, H=4, Dh=32, seed=0)
    out, lse = _gpu(inp, torch.float32, return_lse=True)
    ref, ref_lse = _oracle(inp, return_lse=True)
    assert (out.cpu().double() - ref).abs().max().item() <= F32_MAX_ABS
    assert (lse.cpu().double() - ref_lse).abs().max().item() <= 1e-4
    import os
    import numpy as np
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "c1_seed0.npz"))
    assert np.abs(out.cpu().numpy() - g["out"]).max() <= F32_MAX_ABS


@pytest.mark.parametrize("cfg", [
    dict(B=1, C=3, T=13, H=2, Dh=16, Hkv=1),
    dict(B=2, C=5, T=23, H=4, Dh=64, Hkv=2, validity=True),
    dict(B=1, C=130, T=3, H=2, Dh=128, Hkv=2),
    dict(B=1, C=1, T=40, H=1, Dh=32),
])
def test_fp32_generic_shapes(cfg):
    inp = make_mvpa_inputs(seed=1, table_std=0.3, **cfg)
    out = _gpu(inp, torch.float32)
    assert (out.cpu().double() - _oracle(inp)).abs().max().item() <= F32_MAX_ABS


def test_fp32_flags_and_key_bias():
    inp = make_mvpa_inputs(B=2, C=4, T=15, H=2, Dh=32, seed=4, table_std=0.3)
    d = inp.to("cuda", torch.float32)
    kb = torch.randn(2, 60) * 0.5
    kb[0, 7] = torch.finfo(torch.float32).min
    out = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                key_bias=kb.cuda(), window=3, sm_scale=0.11)
    ref = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                        key_bias=kb, window=3, sm_scale=0.11)
    assert (out.cpu().double() - ref).abs().max().item() <= F32_MAX_ABS
    out = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan, content=False)
    ref = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                        global_att=False)
    assert (out.cpu().double() - ref).abs().max().item() <= F32_MAX_ABS
    out = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan, window=0)
    ref = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan, window=0)
    assert (out.cpu().double() - ref).abs().max().item() <= F32_MAX_ABS


def test_strided_head_interleaved_layout():
    """q/k/v as [B,T,C,H,Dh] views and the output written head-merged, without copies."""
    inp = make_mvpa_inputs(B=2, C=4, T=12, H=4, Dh=32, Hkv=2, seed=6, table_std=0.3)
    d = inp.to("cuda", torch.float32)
    B, H, N, Dh = d.q.shape
    packed = torch.cat([d.q.permute(0, 2, 1, 3).reshape(B, N, -1),
                        d.k.permute(0, 2, 1, 3).reshape(B, N, -1),
                        d.v.permute(0, 2, 1, 3).reshape(B, N, -1)], dim=-1).contiguous()
    e, kv = H * Dh, 2 * Dh
    q = packed[:, :, :e].view(B, N, H, Dh).permute(0, 2, 1, 3)
    k = packed[:, :, e:e + kv].view(B, N, 2, Dh).permute(0, 2, 1, 3)
    v = packed[:, :, e + kv:].view(B, N, 2, Dh).permute(0, 2, 1, 3)
    merged = torch.zeros((B, N, H, Dh), device="cuda")
    mvpa_hip.mvpa_forward(q, k, v, d.u, d.vb, d.z, d.k_time, d.k_chan, out=merged.permute(0, 2, 1, 3))
    ref = _oracle(inp)
    assert (merged.permute(0, 2, 1, 3).cpu().double() - ref).abs().max().item() <= F32_MAX_ABS


def test_bf16_generic_kernel_parity():
    inp = make_mvpa_inputs(B=2, C=8, T=32, H=4, Dh=32, seed=0).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_GENERIC).float().cpu()
    ref = _oracle(inp).float()
    assert (out - ref).abs().max().item() <= BF16_MAX_ABS
    assert _rel_l2(out, ref) <= BF16_REL_L2


def test_masks_are_exact_under_perturbation():
    """Keys that the masks remove must not influence the result at all: outputs stay
    bit-identical when K/V change at causally hidden or invalid keys, and when only K
    changes outside the content window."""
    cfg = dict(B=1, C=6, T=20, H=2, Dh=32, seed=9, table_std=0.3, validity=True)
    inp = make_mvpa_inputs(**cfg)
    inp.chan_valid[0, 2] = False
    base = _gpu(inp, torch.float32)
    C, T = inp.C, inp.T
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    dead = (~inp.chan_valid[0]).nonzero().flatten()
    for t in range(T):
        p.k[:, :, t * C + dead] += 5.0
        p.v[:, :, t * C + dead] -= 5.0
    p.k[:, :, -C:] *= 2.0
    p.v[:, :, -C:] *= 2.0
    out = _gpu(p, torch.float32)
    assert torch.equal(out[:, :, :-C], base[:, :, :-C])
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    p.k[:, :, :C] += 1.0           # time step 0: inside the window only for tq <= 10 and tq == T-1
    out = _gpu(p, torch.float32)
    same = (out == base).flatten(0, 1).all(-1).view(-1, T, C).all(0).all(-1).cpu()
    assert same.tolist() == [not (t <= 10 or t == T - 1) for t in range(T)]


# ------------------------------------------------------------------------------------------
# tiled bf16 MFMA kernel
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("cfg", [dict(B=2, C=8, T=32, H=4, Dh=32), dict(B=1, C=20, T=14, H=2, Hkv=1, Dh=64, validity=True),
                                 dict(B=1, C=5, T=13, H=2, Dh=128)])
def test_fp16_io_on_the_fp32_math_kernel(cfg):
    """fp16 tensors (the reference's kernel takes fp16 or bf16, attentions/attn.py:1064-1066) on
    the fp32-math kernel: inputs rounded to fp16, fp32 arithmetic, one rounding of the output.
    Tolerance: max-abs 2e-3 against the oracle on the same rounded inputs; the log-sum-exp 1e-4."""
    inp = make_mvpa_inputs(seed=5, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.float16)
    out, lse = _gpu(inp, torch.float16, return_lse=True, kernel=mvpa_hip.KERNEL_GENERIC)
    assert out.dtype == torch.float16
    ref, ref_lse = _oracle(inp, return_lse=True)
    assert (out.float().cpu().double() - ref).abs().max().item() <= 2e-3
    assert (lse.cpu().double() - ref_lse).abs().max().item() <= 1e-4


MFMA_SHAPES = [
    dict(B=1, C=8, T=32, H=2, Dh=32),                              # c1's grid, padded 8 -> 32
    dict(B=2, C=64, T=16, H=2, Dh=64),                             # one wave per time step
    dict(B=1, C=32, T=70, H=2, Dh=64),                             # crosses two 32-step slabs
    dict(B=2, C=40, T=20, H=4, Dh=64, Hkv=2, validity=True),       # ragged channels, GQA
    dict(B=1, C=117, T=14, H=2, Dh=64, validity=True),             # c3's channel count
    dict(B=1, C=65, T=40, H=2, Dh=64),                             # just past 64: keys in two parts, far steps, two slabs
    dict(B=2, C=128, T=21, H=4, Dh=64, Hkv=2, validity=True),      # both key parts full, GQA, absent channels
    dict(B=1, C=96, T=45, H=3, Dh=64),                             # second key part half empty; B*H not a multiple of 8
    dict(B=1, C=128, T=6, H=2, Dh=128, Hkv=1),                     # base-model head size
    dict(B=1, C=64, T=13, H=2, Dh=128),
    dict(B=1, C=20, T=37, H=1, Dh=128, validity=True),
    dict(B=1, C=1, T=45, H=2, Dh=32),
    dict(B=3, C=33, T=5, H=3, Dh=32),                              # B*H not a multiple of 8
    dict(B=2, C=16, T=1, H=4, Dh=64),                              # a single time step
    dict(B=4, C=64, T=9, H=4, Dh=64),                              # two (b,h) per XCD: merged tail order
    dict(B=2, C=48, T=11, H=8, Dh=64, Hkv=2),                      # window just vacuous, GQA 4:1
    # far steps (T > 11) on every build of the kernel the dispatcher can pick
    dict(B=1, C=128, T=26, H=2, Dh=128, Hkv=1),                    # <128,4,4,2>: the base model's attention shape, GQA 2:1
    dict(B=1, C=100, T=24, H=4, Dh=128, Hkv=2, validity=True),     # <128,4,4,2>, ragged channels, absent channels
    dict(B=1, C=64, T=30, H=2, Dh=128, Hkv=1),                     # <128,2,4,3>
    dict(B=1, C=48, T=26, H=2, Dh=32),                             # <32,2,8,4>
    dict(B=1, C=100, T=24, H=2, Dh=32, validity=True),             # <32,4,4,4>
    dict(B=1, C=64, T=64, H=3, Dh=64, Hkv=1),                      # MVPFormer-S's attention shape: GQA 3:1, two slabs
    dict(B=1, C=128, T=45, H=2, Dh=128, Hkv=1, validity=True),     # <128,4,4,2> across two 32-step slabs
]


def _check_bf16(out, ref):
    out, ref = out.float().cpu(), ref.float()
    err = (out - ref).abs().max().item()
    rel = _rel_l2(out, ref)
    assert err <= BF16_MAX_ABS and rel <= BF16_REL_L2, f"max-abs {err:.3e}, rel-L2 {rel:.3e}"


@pytest.mark.parametrize("cfg", MFMA_SHAPES)
def test_bf16_mfma_shapes(cfg):
    inp = make_mvpa_inputs(seed=21, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.bfloat16)
    out, lse = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA, return_lse=True)
    ref, ref_lse = _oracle(inp, return_lse=True)
    _check_bf16(out, ref)
    assert (lse.cpu().double() - ref_lse).abs().max().item() <= 3e-2


FP16_MAX_ABS, FP16_REL_L2, FP16_LSE = 5e-4, 1e-3, 1e-3


@pytest.mark.parametrize("cfg", MFMA_SHAPES)
def test_fp16_mfma_shapes(cfg):
    """fp16 tensors on the matrix cores (the general tiled kernel with the fp16 MFMA; the
    reference's kernel takes fp16 or bf16, attentions/attn.py:1064-1066).  Probabilities and the
    far steps' channel factors pass through fp16 (11 significant bits) where the bf16 build has 8,
    so the tolerance against the oracle on the same fp16-rounded inputs is tighter than bf16's:
    max-abs 5e-4, rel-L2 1e-3, log-sum-exp 1e-3 (measured over these shapes: 1.5e-4, 2.9e-4,
    2.5e-4)."""
    inp = make_mvpa_inputs(seed=21, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.float16)
    out, lse = _gpu(inp, torch.float16, kernel=mvpa_hip.KERNEL_MFMA, return_lse=True)
    assert out.dtype == torch.float16
    ref, ref_lse = _oracle(inp, return_lse=True)
    o = out.float().cpu()
    err, rel = (o - ref.float()).abs().max().item(), _rel_l2(o, ref.float())
    assert err <= FP16_MAX_ABS and rel <= FP16_REL_L2, f"max-abs {err:.3e}, rel-L2 {rel:.3e}"
    assert (lse.cpu().double() - ref_lse).abs().max().item() <= FP16_LSE


def test_fp16_dispatch_and_what_it_refuses():
    """fp16 under the default selector takes the matrix-core kernel (bit for bit the forced
    launch); the specialised bf16 builds and the fp8 content term refuse fp16 tensors."""
    cfg = dict(B=1, C=64, T=140, H=2, Dh=64)
    d = make_mvpa_inputs(seed=2, qkv_unit=True, **cfg).to("cuda", torch.float16)
    args = (d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan)
    auto = mvpa_hip.mvpa_forward(*args)
    forced = mvpa_hip.mvpa_forward(*args, kernel=mvpa_hip.KERNEL_MFMA)
    assert torch.equal(auto, forced)
    generic = mvpa_hip.mvpa_forward(*args, kernel=mvpa_hip.KERNEL_GENERIC)
    assert not torch.equal(auto, generic)
    assert (auto.float() - generic.float()).abs().max().item() <= FP16_MAX_ABS
    for kern in (mvpa_hip.KERNEL_MFMA_STEP, mvpa_hip.KERNEL_MFMA_SPLIT):
        with pytest.raises(mvpa_hip.MvpaError):
            mvpa_hip.mvpa_forward(*args, kernel=kern)
    with pytest.raises(mvpa_hip.MvpaError):
        mvpa_hip.mvpa_forward(*args, fp8_qk=True)


# the build of the kernel in which a wave owns a whole time step (head size 64, 33..64 channels);
# the dispatcher picks it from 128 time steps on, the tests force it at every length
STEP_SHAPES = [
    dict(B=2, C=64, T=16, H=2, Dh=64),                             # no far steps but the last-step workgroup
    dict(B=1, C=64, T=40, H=2, Dh=64),                             # far steps, two slabs, T a multiple of 4
    dict(B=2, C=40, T=33, H=4, Hkv=2, Dh=64, validity=True),       # ragged channels, GQA, T-1 a multiple of 4
    dict(B=1, C=33, T=70, H=3, Hkv=1, Dh=64),                      # three slabs; B*H not a multiple of 8
    dict(B=1, C=64, T=134, H=2, Dh=64, validity=True),             # past 128 steps (also the dispatcher's choice)
    dict(B=4, C=64, T=9, H=4, Dh=64),                              # two (b,h) per XCD: merged tail order
    dict(B=2, C=48, T=11, H=8, Dh=64, Hkv=2),                      # window just vacuous
    dict(B=1, C=64, T=64, H=3, Dh=64, Hkv=1),                      # MVPFormer-S's attention shape
    dict(B=1, C=50, T=1, H=2, Dh=64),                              # a single time step
    dict(B=1, C=64, T=2, H=1, Dh=64),
    dict(B=1, C=64, T=5, H=2, Dh=64),
    dict(B=1, C=36, T=6, H=2, Dh=64),                              # T-1 = 5: a tile of one time step
]


@pytest.mark.parametrize("cfg", STEP_SHAPES)
def test_bf16_whole_step_build_shapes(cfg):
    inp = make_mvpa_inputs(seed=27, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.bfloat16)
    out, lse = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_STEP, return_lse=True)
    ref, ref_lse = _oracle(inp, return_lse=True)
    _check_bf16(out, ref)
    assert (lse.cpu().double() - ref_lse).abs().max().item() <= 3e-2


@pytest.mark.parametrize("kw", [dict(window=3), dict(window=0), dict(content=False), dict(window=1),
                                dict(time_bias=False), dict(chan_bias=False), dict(sm_scale=0.05),
                                dict(window=200)])
def test_bf16_whole_step_build_flags(kw):
    inp = make_mvpa_inputs(B=1, C=48, T=45, H=2, Dh=64, seed=28, table_std=0.3,
                           qkv_unit=True).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_STEP, **kw)
    okw = dict(kw)
    if "content" in okw:
        okw["global_att"] = okw.pop("content")
    tb, cb = okw.pop("time_bias", True), okw.pop("chan_bias", True)
    ref_in = inp
    if not tb or not cb:
        import copy
        ref_in = copy.copy(inp)
        if not tb:
            ref_in.k_time = torch.zeros_like(inp.k_time)
        if not cb:
            ref_in.k_chan = torch.zeros_like(inp.k_chan)
    _check_bf16(out, _oracle(ref_in, **okw))


def test_bf16_whole_step_build_large_logits_and_masks():
    """Wide score range (running-max bookkeeping across the window passes and the far phase), and
    masks exact under perturbation, on the whole-time-step build."""
    inp = make_mvpa_inputs(B=1, C=40, T=48, H=2, Dh=64, seed=23, table_std=1.0).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_STEP)
    assert torch.isfinite(out).all()
    _check_bf16(out, _oracle(inp))
    cfg = dict(B=1, C=40, T=20, H=2, Dh=64, seed=9, table_std=0.3, qkv_unit=True, validity=True)
    inp = make_mvpa_inputs(**cfg)
    inp.chan_valid[0, 2] = False
    run = lambda i: _gpu(i, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_STEP)    # noqa: E731
    base = run(inp)
    C, T = inp.C, inp.T
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    dead = (~inp.chan_valid[0]).nonzero().flatten()
    for t in range(T):
        p.k[:, :, t * C + dead] += 5.0
        p.v[:, :, t * C + dead] = 1.0e4
    p.k[:, :, -C:] *= 2.0
    p.v[:, :, -C:] *= 2.0
    assert torch.equal(run(p)[:, :, :-C], base[:, :, :-C])
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    p.k[:, :, :C] += 1.0
    same = (run(p) == base).flatten(0, 1).all(-1).view(-1, T, C).all(0).all(-1).cpu()
    assert same.tolist() == [not (t <= 10 or t == T - 1) for t in range(T)]


def test_whole_step_build_refuses_other_shapes():
    d = make_mvpa_inputs(seed=1, B=1, C=20, T=6, H=1, Dh=64).to("cuda", torch.bfloat16)
    with pytest.raises(mvpa_hip.MvpaError):
        mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan, kernel=mvpa_hip.KERNEL_MFMA_STEP)


# the build of the kernel for 65..128 channels (head size 128: the output columns of a query tile
# split over two waves; head size 64: a workgroup on two time steps): the dispatcher's choice for
# such shapes
SPLIT_SHAPES = [
    dict(B=1, C=128, T=26, H=2, Dh=128, Hkv=1),                    # the base model's attention shape, GQA 2:1
    dict(B=1, C=100, T=24, H=4, Dh=128, Hkv=2, validity=True),     # ragged channels, absent channels
    dict(B=1, C=128, T=45, H=2, Dh=128, Hkv=1, validity=True),     # two 32-step slabs
    dict(B=1, C=65, T=40, H=2, Dh=128),                            # just past 64: three key tiles, one nearly empty
    dict(B=2, C=96, T=13, H=2, Dh=128, Hkv=1),                     # three key tiles exactly; two far steps
    dict(B=1, C=97, T=70, H=3, Dh=128, Hkv=1),                     # four key tiles, one nearly empty; three slabs; B*H odd
    dict(B=4, C=80, T=9, H=4, Dh=128),                             # no far steps; two (b,h) per XCD
    dict(B=1, C=128, T=1, H=2, Dh=128),                            # a single time step
    dict(B=1, C=70, T=2, H=1, Dh=128),
    dict(B=1, C=128, T=12, H=2, Dh=128, Hkv=2),                    # exactly one far step
    # head size 64: a wave owns every output column, a workgroup two time steps
    dict(B=1, C=117, T=14, H=2, Dh=64, validity=True),             # c3's channel count
    dict(B=1, C=65, T=40, H=2, Dh=64),                             # just past 64, two slabs, T even
    dict(B=2, C=128, T=21, H=4, Dh=64, Hkv=2, validity=True),      # T odd: the last workgroup holds one time step
    dict(B=1, C=96, T=45, H=3, Dh=64),                             # a query tile and a key tile without channels; B*H odd
    dict(B=1, C=128, T=70, H=2, Dh=64, Hkv=1),                     # three slabs
    dict(B=1, C=100, T=1, H=2, Dh=64),
    dict(B=1, C=100, T=2, H=2, Dh=64),
    dict(B=4, C=80, T=12, H=4, Dh=64),                             # the last pair (10, 11): one far step for step 10 only
    dict(B=1, C=117, T=13, H=2, Dh=64),                            # pairs (10, 11) and (12): far steps in a workgroup whose partner is the last step
    # 33..64 channels: two key tiles, two query tiles per time step, twice the time steps per workgroup
    dict(B=1, C=64, T=30, H=2, Dh=128, Hkv=1),                     # two time steps per workgroup
    dict(B=1, C=50, T=47, H=4, Dh=128, Hkv=2, validity=True),      # ragged, odd T
    dict(B=1, C=40, T=33, H=3, Dh=64, Hkv=1),                      # four time steps per workgroup, T = 4k + 1
    dict(B=2, C=64, T=15, H=4, Dh=64),                             # T = 4k + 3: the last workgroup holds steps 12, 13, 14
    dict(B=1, C=64, T=70, H=2, Dh=64, validity=True),
    dict(B=1, C=33, T=1, H=2, Dh=64),
]


@pytest.mark.parametrize("cfg", SPLIT_SHAPES)
def test_bf16_column_split_build_shapes(cfg):
    inp = make_mvpa_inputs(seed=29, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.bfloat16)
    out, lse = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_SPLIT, return_lse=True)
    ref, ref_lse = _oracle(inp, return_lse=True)
    _check_bf16(out, ref)
    assert (lse.cpu().double() - ref_lse).abs().max().item() <= 3e-2
    if cfg["C"] > 64 or cfg["Dh"] == 128:                  # the dispatcher picks this build
        assert torch.equal(_gpu(inp, torch.bfloat16), out)


@pytest.mark.parametrize("kw", [dict(window=3), dict(window=0), dict(content=False), dict(window=1),
                                dict(time_bias=False), dict(chan_bias=False), dict(sm_scale=0.05),
                                dict(window=200)])
@pytest.mark.parametrize("dh", [128, 64])
def test_bf16_column_split_build_flags(kw, dh):
    inp = make_mvpa_inputs(B=1, C=72, T=45, H=2, Dh=dh, seed=30, table_std=0.3,
                           qkv_unit=True).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_SPLIT, **kw)
    okw = dict(kw)
    if "content" in okw:
        okw["global_att"] = okw.pop("content")
    tb, cb = okw.pop("time_bias", True), okw.pop("chan_bias", True)
    ref_in = inp
    if not tb or not cb:
        import copy
        ref_in = copy.copy(inp)
        if not tb:
            ref_in.k_time = torch.zeros_like(inp.k_time)
        if not cb:
            ref_in.k_chan = torch.zeros_like(inp.k_chan)
    _check_bf16(out, _oracle(ref_in, **okw))


@pytest.mark.parametrize("dh", [128, 64])
def test_bf16_column_split_build_large_logits_and_masks(dh):
    """Wide score range (running-max bookkeeping across the window steps and the far phase), and
    masks exact under perturbation, on the build for 65..128 channels."""
    inp = make_mvpa_inputs(B=1, C=72, T=48, H=2, Dh=dh, seed=23, table_std=1.0).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_SPLIT)
    assert torch.isfinite(out).all()
    _check_bf16(out, _oracle(inp))
    cfg = dict(B=1, C=100, T=20, H=2, Dh=dh, seed=9, table_std=0.3, qkv_unit=True, validity=True)
    inp = make_mvpa_inputs(**cfg)
    inp.chan_valid[0, 2] = False
    run = lambda i: _gpu(i, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_SPLIT)    # noqa: E731
    base = run(inp)
    C, T = inp.C, inp.T
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    dead = (~inp.chan_valid[0]).nonzero().flatten()
    for t in range(T):
        p.k[:, :, t * C + dead] += 5.0
        p.v[:, :, t * C + dead] = 1.0e4
    p.k[:, :, -C:] *= 2.0
    p.v[:, :, -C:] *= 2.0
    assert torch.equal(run(p)[:, :, :-C], base[:, :, :-C])
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    p.k[:, :, :C] += 1.0
    same = (run(p) == base).flatten(0, 1).all(-1).view(-1, T, C).all(0).all(-1).cpu()
    assert same.tolist() == [not (t <= 10 or t == T - 1) for t in range(T)]


def test_column_split_build_refuses_other_shapes():
    for cfg in (dict(C=32, Dh=128), dict(C=100, Dh=32), dict(C=20, Dh=64)):
        d = make_mvpa_inputs(seed=1, B=1, T=6, H=1, **cfg).to("cuda", torch.bfloat16)
        with pytest.raises(mvpa_hip.MvpaError):
            mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan, kernel=mvpa_hip.KERNEL_MFMA_SPLIT)


@pytest.mark.parametrize("kw", [dict(window=3), dict(window=0), dict(content=False),
                                dict(time_bias=False), dict(chan_bias=False), dict(sm_scale=0.05)])
def test_bf16_mfma_flags(kw):
    inp = make_mvpa_inputs(B=1, C=24, T=40, H=2, Dh=64, seed=22, table_std=0.3,
                           qkv_unit=True).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA, **kw)
    okw = dict(kw)
    if "content" in okw:
        okw["global_att"] = okw.pop("content")
    tb, cb = okw.pop("time_bias", True), okw.pop("chan_bias", True)
    ref_in = inp
    if not tb or not cb:
        import copy
        ref_in = copy.copy(inp)
        if not tb:
            ref_in.k_time = torch.zeros_like(inp.k_time)
        if not cb:
            ref_in.k_chan = torch.zeros_like(inp.k_chan)
    _check_bf16(out, _oracle(ref_in, **okw))


def test_bf16_mfma_large_logits():
    """Wide score range (q,k,v ~ N(0,1), tables std 1): running-max bookkeeping of the far and
    near paths must not overflow or lose rows."""
    inp = make_mvpa_inputs(B=1, C=16, T=48, H=2, Dh=32, seed=23, table_std=1.0).round_to(torch.bfloat16)
    out = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA)
    assert torch.isfinite(out).all()
    _check_bf16(out, _oracle(inp))


def test_bf16_mfma_masks_exact_under_perturbation():
    cfg = dict(B=1, C=40, T=20, H=2, Dh=64, seed=9, table_std=0.3, qkv_unit=True, validity=True)
    inp = make_mvpa_inputs(**cfg)
    inp.chan_valid[0, 2] = False
    run = lambda i: _gpu(i, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA)
    base = run(inp)
    C, T = inp.C, inp.T
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    dead = (~inp.chan_valid[0]).nonzero().flatten()
    for t in range(T):
        p.k[:, :, t * C + dead] += 5.0
        p.v[:, :, t * C + dead] = 1.0e4               # absent channels may hold any finite value
    p.k[:, :, -C:] *= 2.0
    p.v[:, :, -C:] *= 2.0
    out = run(p)
    assert torch.equal(out[:, :, :-C], base[:, :, :-C])
    p = make_mvpa_inputs(**cfg)
    p.chan_valid = inp.chan_valid
    p.k[:, :, :C] += 1.0
    out = run(p)
    same = (out == base).flatten(0, 1).all(-1).view(-1, T, C).all(0).all(-1).cpu()
    assert same.tolist() == [not (t <= 10 or t == T - 1) for t in range(T)]


@pytest.mark.parametrize("cfg", [
    dict(B=2, C=117, T=30, H=2, Dh=64),                            # keys in two parts (KH = 2), far steps
    dict(B=2, C=128, T=14, H=4, Dh=64, Hkv=2),
    dict(B=2, C=128, T=26, H=2, Dh=128, Hkv=1),                    # one wave on all four key tiles
])
def test_bf16_mfma_whole_key_part_absent(cfg):
    """Every channel from 64 up absent in one sample (a subject with 64 electrodes padded into a
    wider batch): the waves that own the second half of the keys see no valid key at all and must
    contribute exactly nothing - finite output, equal to the oracle."""
    inp = make_mvpa_inputs(seed=33, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.bfloat16)
    valid = torch.ones(cfg["B"], cfg["C"], dtype=torch.bool)
    valid[0, 64:] = False
    valid[1, :64] = False                                          # and the first half, in the other sample
    valid[1, 70] = True
    inp.chan_valid = valid
    out, lse = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA, return_lse=True)
    live = valid[:, None, None, :].expand(-1, 1, cfg["T"], -1).reshape(cfg["B"], 1, -1, 1)
    assert torch.isfinite(out.float().cpu()[live.expand_as(out)]).all()
    ref, ref_lse = _oracle(inp, return_lse=True)
    _check_bf16(out.float().cpu() * live, ref * live)
    assert ((lse.cpu().double() - ref_lse) * live[..., 0]).abs().max().item() <= 3e-2


@pytest.mark.parametrize("cfg,n,ring", [
    (dict(B=1, C=117, T=24, H=2, Hkv=2, Dh=64), 3, False),
    (dict(B=1, C=128, T=40, H=2, Hkv=1, Dh=128), 5, False),        # the 8-wave key-run build at Dh 128
    (dict(B=1, C=128, T=40, H=2, Hkv=1, Dh=128), 5, True),
])
def test_last_step_whole_key_part_absent(cfg, n, ring):
    """The same for a decoding step cut into key runs (and on a ring of slots): against the oracle's
    last time step."""
    inp = make_mvpa_inputs(seed=35, table_std=0.3, qkv_unit=True, **cfg).round_to(torch.bfloat16)
    B, C, T, Hkv, Dh = cfg["B"], cfg["C"], cfg["T"], cfg["Hkv"], cfg["Dh"]
    valid = torch.ones(B, C, dtype=torch.bool)
    valid[0, 64:] = False
    inp.chan_valid = valid
    ref = _oracle(inp)[:, :, -C:].float()
    d = inp.to("cuda", torch.bfloat16)
    k, v, head_t = d.k, d.v, None
    if ring:
        head = 17
        slot = torch.arange(T, device="cuda")
        step_of_slot = T - 1 - (head - slot) % T
        k = d.k.view(B, Hkv, T, C, Dh)[:, :, step_of_slot].reshape(B, Hkv, T * C, Dh).contiguous()
        v = d.v.view(B, Hkv, T, C, Dh)[:, :, step_of_slot].reshape(B, Hkv, T * C, Dh).contiguous()
        head_t = torch.tensor([head], dtype=torch.int32, device="cuda")
    got = mvpa_hip.mvpa_forward(d.q[:, :, -C:], k, v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                chan_valid=d.chan_valid, last_step_only=True, key_splits=n,
                                ring_head=head_t).float().cpu()
    live = valid[:, None, :, None]
    assert torch.isfinite(got[live.expand_as(got)]).all()
    _check_bf16(got * live, ref * live)


# ------------------------------------------------------------------------------------------
# gathers of the matrix-core kernel itself, on index-revealing inputs
# ------------------------------------------------------------------------------------------
# q = 0 and u = 0 switch the content term off.  One bias vector is a unit vector and ONE row j* of
# its table holds a large value in that coordinate, so the soft-max puts all its weight on the
# keys whose gathered row is j* (every other key is down by e^-64).  V codes the key's channel
# (or time step) one-hot, so the output names the keys that got the weight: the expected output is
# written down from the closed forms C-1-|cq-ck| and T-1-(tq-tk) (layers/mvpa.py:127-159) and an
# index that is off by one anywhere in the kernel moves ones to other columns.  Head g tests row
# j* = rows[g] (the tables are per kv head).

GATHER_SHAPES = [
    dict(C=64, T=40, Dh=64),        # <64,2,4,4>: split last step, far steps, two slabs
    dict(C=117, T=14, Dh=64),       # keys in two parts
    dict(C=128, T=40, Dh=128),      # one wave on four key tiles
    dict(C=48, T=40, Dh=32),
    dict(C=20, T=70, Dh=64),        # 8 time steps per workgroup, three slabs
    dict(C=100, T=36, Dh=32),
]
PEAK = 64.0


def _gather_case(C, T, Dh, rows, axis):
    """Inputs (fp32, exactly representable in bf16) whose output reveals the gathered row."""
    H = len(rows)
    N = T * C
    q = torch.zeros(1, H, N, Dh)
    k = torch.zeros(1, H, N, Dh)
    zero = torch.zeros(H, Dh)
    unit = torch.zeros(H, Dh)
    unit[:, 0] = 1.0
    k_time, k_chan = torch.zeros(H, T, Dh), torch.zeros(H, C, Dh)
    tab = k_chan if axis == "chan" else k_time
    for g, j in enumerate(rows):
        tab[g, j, 0] = PEAK
    n = torch.arange(N)
    code = (n % C) if axis == "chan" else (n // C)
    v = torch.zeros(1, H, N, Dh)
    v[0, :, n, code % Dh] = 1.0
    return q, k, v, zero, unit, k_time, k_chan


GATHER_CASES = [(c, "KERNEL_MFMA") for c in GATHER_SHAPES] + [
    (dict(C=64, T=40, Dh=64), "KERNEL_MFMA_STEP"), (dict(C=40, T=70, Dh=64), "KERNEL_MFMA_STEP"),
    (dict(C=128, T=40, Dh=128), "KERNEL_MFMA_SPLIT"), (dict(C=70, T=70, Dh=128), "KERNEL_MFMA_SPLIT"),
    (dict(C=117, T=41, Dh=64), "KERNEL_MFMA_SPLIT")]
_gather_id = lambda c: "C{C}T{T}D{Dh}".format(**c) if isinstance(c, dict) else c      # noqa: E731


@pytest.mark.parametrize("cfg,kern", GATHER_CASES, ids=_gather_id)
def test_mfma_channel_gather_is_exact(cfg, kern):
    C, T, Dh = cfg["C"], cfg["T"], cfg["Dh"]
    cq, ck = torch.arange(C)[:, None], torch.arange(C)[None, :]
    onehot = torch.zeros(C, Dh)
    onehot[torch.arange(C), torch.arange(C) % Dh] = 1.0
    for r0 in range(0, C, 16):
        rows = list(range(r0, min(C, r0 + 16)))
        q, k, v, zero, unit, k_time, k_chan = _gather_case(C, T, Dh, rows, "chan")
        out = mvpa_hip.mvpa_forward(*(t.cuda().bfloat16() for t in (q, k, v, zero, zero, unit, k_time, k_chan)),
                                    sm_scale=1.0, kernel=getattr(mvpa_hip, kern)).float().cpu()
        for g, j in enumerate(rows):
            hit = (C - 1 - (cq - ck).abs()) == j                  # keys whose gathered row is j*
            w = torch.where(hit.any(1, keepdim=True), hit, torch.ones_like(hit)).float()
            want = (w / w.sum(1, keepdim=True)) @ onehot          # [C, Dh], the same for every tq
            got = out[0, g].view(T, C, Dh)
            assert (got - want[None]).abs().max().item() <= 1e-2, (j, (got - want[None]).abs().max().item())


@pytest.mark.parametrize("cfg,kern", GATHER_CASES, ids=_gather_id)
def test_mfma_time_gather_is_exact(cfg, kern):
    C, T, Dh = cfg["C"], cfg["T"], cfg["Dh"]
    for r0 in range(0, T, 16):
        rows = list(range(r0, min(T, r0 + 16)))
        q, k, v, zero, unit, k_time, k_chan = _gather_case(C, T, Dh, rows, "time")
        out = mvpa_hip.mvpa_forward(*(t.cuda().bfloat16() for t in (q, k, v, zero, unit, zero, k_time, k_chan)),
                                    sm_scale=1.0, kernel=getattr(mvpa_hip, kern)).float().cpu()
        for g, j in enumerate(rows):
            got = out[0, g].view(T, C, Dh)
            for tq in range(T):
                tk = tq - (T - 1 - j)                             # the key step whose gathered row is j*
                want = torch.zeros(Dh)
                if tk >= 0:
                    want[tk % Dh] = 1.0
                else:                                             # row j* out of reach: uniform over tk <= tq
                    for t in range(tq + 1):
                        want[t % Dh] += 1.0 / (tq + 1)
                err = (got[tq] - want[None]).abs().max().item()
                assert err <= 1e-2, (j, tq, err)


@pytest.mark.parametrize("cfg,n,head", [
    (dict(C=64, T=40, Dh=64), 4, 13),
    (dict(C=128, T=70, Dh=128), 5, 33),        # runs longer than a slab, the ring wraps inside a run
    (dict(C=20, T=45, Dh=32), 1, 44),
])
def test_mfma_time_gather_on_a_ring_is_exact(cfg, n, head):
    """Decoding step on a ring of slots: the table row of slot s is (s - head - 1) mod T, read per
    slab inside the kernel.  The step that holds row j* must get the weight wherever the ring
    stands."""
    C, T, Dh = cfg["C"], cfg["T"], cfg["Dh"]
    slot = torch.arange(T)
    step_of_slot = T - 1 - (head - slot) % T
    head_t = torch.tensor([head], dtype=torch.int32, device="cuda")
    for r0 in range(0, T, 16):
        rows = list(range(r0, min(T, r0 + 16)))
        H = len(rows)
        q, k, v, zero, unit, k_time, k_chan = _gather_case(C, T, Dh, rows, "time")
        v_ring = v.view(1, H, T, C, Dh)[:, :, step_of_slot].reshape(1, H, T * C, Dh)
        args = [t.cuda().bfloat16() for t in (q[:, :, -C:], k, v_ring, zero, unit, zero, k_time, k_chan)]
        out = mvpa_hip.mvpa_forward(*args, sm_scale=1.0, last_step_only=True, key_splits=n,
                                    ring_head=head_t).float().cpu()
        for g, j in enumerate(rows):
            want = torch.zeros(Dh)
            want[j % Dh] = 1.0                                    # tq = T-1: row j* belongs to key step j*
            assert (out[0, g] - want[None]).abs().max().item() <= 1e-2, j


def test_bf16_mfma_strided_layout_and_auto_dispatch():
    inp = make_mvpa_inputs(B=2, C=16, T=12, H=4, Dh=64, Hkv=2, seed=6, table_std=0.3,
                           qkv_unit=True).round_to(torch.bfloat16)
    d = inp.to("cuda", torch.bfloat16)
    B, H, N, Dh = d.q.shape
    packed = torch.cat([d.q.permute(0, 2, 1, 3).reshape(B, N, -1),
                        d.k.permute(0, 2, 1, 3).reshape(B, N, -1),
                        d.v.permute(0, 2, 1, 3).reshape(B, N, -1)], dim=-1).contiguous()
    e, kv = H * Dh, 2 * Dh
    q = packed[:, :, :e].view(B, N, H, Dh).permute(0, 2, 1, 3)
    k = packed[:, :, e:e + kv].view(B, N, 2, Dh).permute(0, 2, 1, 3)
    v = packed[:, :, e + kv:].view(B, N, 2, Dh).permute(0, 2, 1, 3)
    merged = torch.zeros((B, N, H, Dh), device="cuda", dtype=torch.bfloat16)
    import ctypes
    a = mvpa_hip.make_args(q, k, v, merged.permute(0, 2, 1, 3), d.u, d.vb, d.z, d.k_time, d.k_chan,
                           T=inp.T, C=inp.C, sm_scale=Dh ** -0.5)
    assert mvpa_hip.load_library().mvpa_select_kernel(ctypes.byref(a)) == mvpa_hip.KERNEL_MFMA
    mvpa_hip.mvpa_forward(q, k, v, d.u, d.vb, d.z, d.k_time, d.k_chan, out=merged.permute(0, 2, 1, 3))
    _check_bf16(merged.permute(0, 2, 1, 3), _oracle(inp))


@pytest.mark.parametrize("kern", ["KERNEL_AUTO", "KERNEL_MFMA"])
def test_bf16_config2_full_size(kern):
    """Config c2 (B4 C64 T128 H16 Dh64) on the build the library picks for it (a wave owns a whole
    time step) and on the general kernel: two heads against the oracle, the rest through
    size-independent properties."""
    kern = getattr(mvpa_hip, kern)
    inp = make_mvpa_inputs(B=4, C=64, T=128, H=16, Dh=64, seed=0, qkv_unit=True).round_to(torch.bfloat16)
    d = inp.to("cuda", torch.bfloat16)
    out = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                kernel=kern)
    heads = [(0, 0), (3, 15)]
    ref = _oracle(inp, dtype=torch.float32, heads=heads, q_block=1024)
    for (b, h) in heads:
        _check_bf16(out[b, h], ref[b, h])
    # V == 1 -> every output is 1 (rows of P sum to one)
    ones = torch.ones_like(d.v)
    o1 = mvpa_hip.mvpa_forward(d.q, d.k, ones, d.u, d.vb, d.z, d.k_time, d.k_chan, kernel=kern).float()
    assert (o1 - 1).abs().max().item() <= 1e-2
    # causality, bit exact: changing the last 16 time steps leaves earlier rows untouched
    k2, v2 = d.k.clone(), d.v.clone()
    k2[:, :, -16 * 64:] *= -1.5
    v2[:, :, -16 * 64:] += 1.0
    o2 = mvpa_hip.mvpa_forward(d.q, k2, v2, d.u, d.vb, d.z, d.k_time, d.k_chan, kernel=kern)
    assert torch.equal(o2[:, :, :-16 * 64], out[:, :, :-16 * 64])
    # agreement with the fp32-math generic kernel on every head
    og = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                               kernel=mvpa_hip.KERNEL_GENERIC)
    _check_bf16(out, og.float().cpu())


@pytest.mark.parametrize("kern", ["KERNEL_AUTO", "KERNEL_MFMA"])
def test_bf16_config3_irregular_channels(kern):
    """Config c3 (B8 C117 T256 H16 Dh64, per-sample channel validity) on the build the library
    picks for it (65..128 channels: a workgroup on two time steps) and on the general kernel:
    sampled query rows of one head against the oracle, masks through bit-exact perturbation."""
    kern = getattr(mvpa_hip, kern)
    inp = make_mvpa_inputs(B=8, C=117, T=256, H=16, Dh=64, seed=0, qkv_unit=True,
                           validity=True).round_to(torch.bfloat16)
    d = inp.to("cuda", torch.bfloat16)
    out = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                chan_valid=d.chan_valid, kernel=kern)
    C = 117
    ranges = [(0, 2 * C), (100 * C, 101 * C), (255 * C, 256 * C)]
    ref = _oracle(inp, dtype=torch.float32, heads=[(5, 7)], q_ranges=ranges, q_block=256)
    for (r0, r1) in ranges:
        _check_bf16(out[5, 7, r0:r1], ref[5, 7, r0:r1])
    # invalid channels and future keys never matter
    dead = (~d.chan_valid)[:, None, None, :, None]            # [B,1,1,C,1]
    seven = torch.tensor(7.0, dtype=torch.bfloat16, device="cuda")
    big = torch.tensor(-3.0e4, dtype=torch.bfloat16, device="cuda")
    k2 = torch.where(dead, seven, d.k.view(8, 16, 256, C, 64)).view(8, 16, 256 * C, 64)
    v2 = torch.where(dead, big, d.v.view(8, 16, 256, C, 64)).view(8, 16, 256 * C, 64)
    o2 = mvpa_hip.mvpa_forward(d.q, k2, v2, d.u, d.vb, d.z, d.k_time, d.k_chan,
                               chan_valid=d.chan_valid, kernel=kern)
    assert torch.equal(o2, out)


# fp8 (e4m3) content term: 3 mantissa bits on q' and k.  Rounding both factors to e4m3 perturbs a
# content score by about 2.5 % of the score's own spread, so the stated tolerance scales with how
# wide the content logits are: unit-variance logits (q, k ~ N(0,1), Dh = 64) versus the narrow
# logits of the benchmark distribution (q, k ~ N(0,1)/sqrt(Dh)).
FP8_TOL = {False: dict(max_abs=1.2e-1, rel_l2=6e-2), True: dict(max_abs=2e-2, rel_l2=6e-3)}


@pytest.mark.parametrize("cfg", [
    dict(B=2, C=64, T=24, H=4, Dh=64, Hkv=2, qkv_unit=False, table_std=0.3),
    dict(B=1, C=117, T=14, H=2, Dh=64, qkv_unit=True, table_std=0.3, validity=True),
    dict(B=1, C=128, T=13, H=2, Dh=128, Hkv=1, qkv_unit=False, table_std=0.3),
])
def test_fp8_qk_within_stated_tolerance(cfg):
    """QK^T of the content term in fp8 e4m3 with per-head amax scales (biases, soft-max and PV
    unchanged).  The reference has no fp8 path; the tolerance against the fp64 oracle is this
    build's own statement."""
    inp = make_mvpa_inputs(seed=31, **cfg).round_to(torch.bfloat16)
    ref = _oracle(inp).float()
    o8 = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA, fp8_qk=True).float().cpu()
    o16 = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA).float().cpu()
    assert not torch.equal(o8, o16)                     # the fp8 path really ran
    err, rel = (o8 - ref).abs().max().item(), _rel_l2(o8, ref)
    tol = FP8_TOL[cfg["qkv_unit"]]
    print(f"fp8 QK^T: max-abs {err:.3e} rel-L2 {rel:.3e} (bf16: {(o16 - ref).abs().max().item():.3e}, {_rel_l2(o16, ref):.3e})")
    assert err <= tol["max_abs"] and rel <= tol["rel_l2"], f"max-abs {err:.3e}, rel-L2 {rel:.3e}"


@pytest.mark.parametrize("cfg", [
    dict(B=1, C=128, T=26, H=2, Dh=128, Hkv=1, qkv_unit=False, table_std=0.3),             # far steps too
    dict(B=1, C=100, T=24, H=4, Dh=128, Hkv=2, qkv_unit=True, table_std=0.3, validity=True),
    dict(B=2, C=80, T=9, H=2, Dh=128, qkv_unit=False, table_std=0.3),                      # window steps only
])
def test_fp8_qk_on_the_column_split_build(cfg):
    """The fp8 content term on the build with the output columns split over two waves (the
    library's choice for head size 128 with 65..128 channels): the same stated tolerance against
    the oracle as on the general kernel, and agreement with the general kernel's fp8 result to
    bf16 rounding (both round the same q' and k' to e4m3)."""
    inp = make_mvpa_inputs(seed=33, **cfg).round_to(torch.bfloat16)
    ref = _oracle(inp).float()
    o8 = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_SPLIT, fp8_qk=True).float().cpu()
    o16 = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA_SPLIT).float().cpu()
    og8 = _gpu(inp, torch.bfloat16, kernel=mvpa_hip.KERNEL_MFMA, fp8_qk=True).float().cpu()
    auto8 = _gpu(inp, torch.bfloat16, fp8_qk=True).float().cpu()
    assert not torch.equal(o8, o16)                     # the fp8 path really ran
    assert torch.equal(auto8, o8)                       # and it is the build the library picks
    B, T, C = cfg["B"], cfg["T"], cfg["C"]
    live = torch.ones_like(o8[..., :1]) if inp.chan_valid is None else \
        inp.chan_valid[:, None, None, :, None].expand(B, 1, T, C, 1).reshape(B, 1, -1, 1).float()
    err, rel = ((o8 - ref) * live).abs().max().item(), _rel_l2(o8 * live, ref * live)
    tol = FP8_TOL[cfg["qkv_unit"]]
    assert err <= tol["max_abs"] and rel <= tol["rel_l2"], f"max-abs {err:.3e}, rel-L2 {rel:.3e}"
    assert ((o8 - og8) * live).abs().max().item() <= 2e-2


@pytest.mark.parametrize("cfg", [dict(B=2, C=40, T=9, H=4, Hkv=2, Dh=64), dict(B=1, C=128, T=5, H=2, Hkv=1, Dh=128)])
def test_fp8_prepare_scales_and_rounded_keys(cfg):
    """mvpa_fp8_prepare: the per-head scales are max|q+u| * s*log2(e)/224 and max|k| / 224, and the
    e4m3 copy of the keys is k * (1/k_scale) rounded to nearest even, byte for byte what torch's
    float8_e4m3fn conversion gives - on strided views of a fused projection, as the layer passes
    them."""
    import ctypes
    lib = mvpa_hip.load_library()
    B, C, T, H, Hkv, Dh = (cfg[k] for k in ("B", "C", "T", "H", "Hkv", "Dh"))
    N = T * C
    torch.manual_seed(17)
    qkv = (torch.randn(B, N, (H + 2 * Hkv) * Dh, device="cuda") * 1.7).to(torch.bfloat16)
    q = qkv[:, :, :H * Dh].view(B, N, H, Dh).permute(0, 2, 1, 3)
    k = qkv[:, :, H * Dh:(H + Hkv) * Dh].view(B, N, Hkv, Dh).permute(0, 2, 1, 3)
    v = qkv[:, :, (H + Hkv) * Dh:].view(B, N, Hkv, Dh).permute(0, 2, 1, 3)
    u = (torch.randn(Hkv, Dh, device="cuda") * 0.5).to(torch.bfloat16)
    tab = torch.zeros(Hkv, max(T, C), Dh, dtype=torch.bfloat16, device="cuda")
    out = torch.empty((B, H, N, Dh), dtype=torch.bfloat16, device="cuda")
    s = Dh ** -0.5
    a = mvpa_hip.make_args(q, k, v, out, u, u, u, tab, tab, T=T, C=C, sm_scale=s)
    qs = torch.empty(H, dtype=torch.float32, device="cuda")
    ks = torch.empty(Hkv, dtype=torch.float32, device="cuda")
    k8 = torch.zeros((B, Hkv, N, Dh), dtype=torch.uint8, device="cuda")
    assert lib.mvpa_fp8_prepare(ctypes.byref(a), qs.data_ptr(), ks.data_ptr(), k8.data_ptr(),
                                torch.cuda.current_stream().cuda_stream) == 0
    qf = q.float() + u.float().repeat_interleave(H // Hkv, 0)[None, :, None, :]
    want_q = qf.abs().amax(dim=(0, 2, 3)) * torch.tensor(a.sm_scale * 1.4426950408889634 / 224.0, dtype=torch.float64).float().cuda()
    want_k = k.float().abs().amax(dim=(0, 2, 3)) / 224.0
    assert torch.allclose(qs, want_q, rtol=2e-7, atol=0) and torch.equal(ks, want_k)
    want8 = (k.float() * (1.0 / ks)[None, :, None, None]).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(k8, want8)
    # scales only
    assert lib.mvpa_fp8_prepare(ctypes.byref(a), qs.data_ptr(), ks.data_ptr(), None,
                                torch.cuda.current_stream().cuda_stream) == 0
    assert torch.equal(ks, want_k)


def test_fp8_needs_mfma_kernel():
    inp = make_mvpa_inputs(B=1, C=4, T=6, H=1, Dh=32, seed=1)
    d = inp.to("cuda", torch.float32)
    with pytest.raises(mvpa_hip.MvpaError):
        mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan, fp8_qk=True)


LAST_STEP_SHAPES = [
    dict(B=2, C=64, T=17, H=4, Hkv=2, Dh=64),      # split last step (two key steps per barrier), odd T
    dict(B=1, C=117, T=12, H=2, Hkv=2, Dh=64),     # keys in two parts
    dict(B=2, C=20, T=40, H=2, Hkv=1, Dh=64),      # 8 waves = 8 time steps per workgroup: 7 of them idle
    dict(B=1, C=64, T=9, H=2, Hkv=2, Dh=128),
    dict(B=3, C=8, T=1, H=1, Hkv=1, Dh=32),        # nothing cached yet
]


@pytest.mark.parametrize("cfg", LAST_STEP_SHAPES, ids=lambda c: "B{B}C{C}T{T}H{H}D{Dh}".format(**c))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
def test_last_step_only_equals_last_rows_of_full_forward(cfg, dtype):
    """MVPA_FLAG_LAST_STEP (one step of incremental decoding: C queries against T*C cached keys)
    gives the rows of the last time step of the full forward: the same kernel code runs on the
    same operands, so bit for bit, output and log-sum-exp."""
    inp = make_mvpa_inputs(seed=17, qkv_unit=True, **cfg).to("cuda", dtype)
    C = cfg["C"]
    tabs = (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)
    kern = mvpa_hip.KERNEL_GENERIC if dtype == torch.float32 else mvpa_hip.KERNEL_MFMA
    full, lse_full = mvpa_hip.mvpa_forward(inp.q, inp.k, inp.v, *tabs, return_lse=True, kernel=kern)
    q_last = inp.q[:, :, -C:]
    step, lse_step = mvpa_hip.mvpa_forward(q_last, inp.k, inp.v, *tabs, return_lse=True,
                                           last_step_only=True, key_splits=1)
    assert step.shape == q_last.shape and lse_step.shape == q_last.shape[:3]
    assert torch.equal(step, full[:, :, -C:])
    assert torch.equal(lse_step, lse_full[:, :, -C:])


SPLIT_CASES = [
    (dict(B=2, C=64, T=17, H=4, Hkv=2, Dh=64), 2),      # runs of 9 and 8 steps
    (dict(B=2, C=64, T=17, H=4, Hkv=2, Dh=64), 17),     # one key step per run
    (dict(B=1, C=117, T=45, H=2, Hkv=2, Dh=64), 4),     # keys in two parts, runs 12+12+12+9
    (dict(B=2, C=20, T=70, H=2, Hkv=1, Dh=64), 3),      # runs longer than a 32-step slab
    (dict(B=1, C=128, T=40, H=2, Hkv=1, Dh=128), 5),
    (dict(B=1, C=64, T=33, H=2, Hkv=2, Dh=128), None),  # the binding's own choice
    (dict(B=3, C=8, T=24, H=2, Hkv=1, Dh=32), 6),
]


@pytest.mark.parametrize("cfg,n", SPLIT_CASES, ids=lambda c: "B{B}C{C}T{T}H{H}D{Dh}".format(**c) if isinstance(c, dict) else f"n{c}")
@pytest.mark.parametrize("fp8", [False, True, "fp16"], ids=["bf16", "fp8qk", "fp16"])
def test_last_step_key_splits_match_unsplit(cfg, n, fp8):
    """The key steps of a last-step launch cut into runs, each on its own workgroups, merged by the
    second kernel: within bf16 rounding of the one-workgroup result (the partial outputs pass
    through bf16; through fp16 for fp16 tensors), log-sum-exp to 1e-3, with some channels absent."""
    dtype = torch.float16 if fp8 == "fp16" else torch.bfloat16
    fp8 = fp8 is True
    inp = make_mvpa_inputs(seed=23, qkv_unit=True, **cfg).to("cuda", dtype)
    C = cfg["C"]
    valid = torch.ones(cfg["B"], C, dtype=torch.bool, device="cuda")
    valid[:, 1::5] = False
    tabs = (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)
    q_last = inp.q[:, :, -C:]
    kw = dict(return_lse=True, last_step_only=True, chan_valid=valid, fp8_qk=fp8)
    ref, lse_ref = mvpa_hip.mvpa_forward(q_last, inp.k, inp.v, *tabs, key_splits=1, **kw)
    got, lse_got = mvpa_hip.mvpa_forward(q_last, inp.k, inp.v, *tabs, key_splits=n, **kw)
    if n is None:
        assert mvpa_hip.default_key_splits(cfg["B"], cfg["H"], cfg["T"]) > 1
    err = (got.float() - ref.float()).abs().max().item()
    rel = ((got.float() - ref.float()).norm() / ref.float().norm()).item()
    assert err <= 2e-2 and rel <= 5e-3, (err, rel)
    assert (lse_got - lse_ref).abs().max().item() <= 1e-3


def test_key_splits_rejected_where_they_make_no_sense():
    d = make_mvpa_inputs(seed=1, B=1, C=8, T=6, H=1, Hkv=1, Dh=64).to("cuda", torch.bfloat16)
    tabs = (d.u, d.vb, d.z, d.k_time, d.k_chan)
    with pytest.raises(AssertionError):    # 4 runs of ceil(6/4) = 2 steps: the last one is empty
        mvpa_hip.mvpa_forward(d.q[:, :, -8:], d.k, d.v, *tabs, last_step_only=True, key_splits=4)
    with pytest.raises(AssertionError):    # more runs than key steps
        mvpa_hip.mvpa_forward(d.q[:, :, -8:], d.k, d.v, *tabs, last_step_only=True, key_splits=7)


@pytest.mark.parametrize("cfg,n,head", [
    (dict(B=2, C=64, T=17, H=4, Hkv=2, Dh=64), 1, 5),
    (dict(B=2, C=64, T=40, H=4, Hkv=2, Dh=64), 4, 39),      # head on the last slot: ring order = time order
    (dict(B=1, C=117, T=45, H=2, Hkv=2, Dh=64), 4, 0),
    (dict(B=1, C=128, T=70, H=2, Hkv=1, Dh=128), 5, 33),    # runs longer than a 32-step slab, wrap inside a run
    (dict(B=3, C=8, T=24, H=2, Hkv=1, Dh=32), None, 23),
])
def test_last_step_on_a_ring_of_slots(cfg, n, head):
    """MVPA_FLAG_RING: the cached time steps sit in the slots of a ring, the newest one in slot
    `head` (read from device memory by the kernel).  Same result as the same steps in time order,
    to bf16 rounding (the key steps are visited in another order)."""
    inp = make_mvpa_inputs(seed=29, qkv_unit=True, **cfg).to("cuda", torch.bfloat16)
    B, C, T, Hkv, Dh = cfg["B"], cfg["C"], cfg["T"], cfg["Hkv"], cfg["Dh"]
    tabs = (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)
    q_last = inp.q[:, :, -C:]
    ref, lse_ref = mvpa_hip.mvpa_forward(q_last, inp.k, inp.v, *tabs, return_lse=True, last_step_only=True, key_splits=1)
    # slot s holds the step that is (head - s) mod T steps older than the newest one (time index T-1)
    slot = torch.arange(T, device="cuda")
    step_of_slot = T - 1 - (head - slot) % T
    k5, v5 = inp.k.view(B, Hkv, T, C, Dh), inp.v.view(B, Hkv, T, C, Dh)
    k_ring = k5[:, :, step_of_slot].reshape(B, Hkv, T * C, Dh).contiguous()
    v_ring = v5[:, :, step_of_slot].reshape(B, Hkv, T * C, Dh).contiguous()
    head_t = torch.tensor([head], dtype=torch.int32, device="cuda")
    got, lse_got = mvpa_hip.mvpa_forward(q_last, k_ring, v_ring, *tabs, return_lse=True, last_step_only=True,
                                         key_splits=n, ring_head=head_t)
    err = (got.float() - ref.float()).abs().max().item()
    rel = ((got.float() - ref.float()).norm() / ref.float().norm()).item()
    assert err <= 2e-2 and rel <= 5e-3, (err, rel)
    assert (lse_got - lse_ref).abs().max().item() <= 1e-3
    # the head is read at run time: moving it (and the slots with it) needs no new arguments
    head_t.fill_((head + 3) % T)
    step_of_slot = T - 1 - ((head + 3) % T - slot) % T
    k_ring.copy_(k5[:, :, step_of_slot].reshape(B, Hkv, T * C, Dh))
    v_ring.copy_(v5[:, :, step_of_slot].reshape(B, Hkv, T * C, Dh))
    got2 = mvpa_hip.mvpa_forward(q_last, k_ring, v_ring, *tabs, last_step_only=True, key_splits=n, ring_head=head_t)
    assert (got2.float() - ref.float()).abs().max().item() <= 2e-2


def test_decoding_step_at_base_model_size_matches_the_full_forward():
    """The base model's attention shape (B1 H16 Hkv8 C128 T512 Dh128): one decoding step with the
    binding's own key runs (16 of 32 steps, the 8-wave key-split build) and on a ring of slots,
    against the last time step of the full forward."""
    cfg = dict(B=1, C=128, T=512, H=16, Hkv=8, Dh=128)
    inp = make_mvpa_inputs(seed=41, **cfg).to("cuda", torch.bfloat16)
    C, T = cfg["C"], cfg["T"]
    tabs = (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)
    full, lse_full = mvpa_hip.mvpa_forward(inp.q, inp.k, inp.v, *tabs, return_lse=True)
    ref, lse_ref = full[:, :, -C:].float(), lse_full[:, :, -C:]
    q_last = inp.q[:, :, -C:]
    assert mvpa_hip.default_key_splits(1, 16, T) == 16
    got, lse_got = mvpa_hip.mvpa_forward(q_last, inp.k, inp.v, *tabs, return_lse=True, last_step_only=True)
    assert (got.float() - ref).abs().max().item() <= 2e-2
    assert ((got.float() - ref).norm() / ref.norm()).item() <= 5e-3
    assert (lse_got - lse_ref).abs().max().item() <= 2e-3
    head = 200
    slot = torch.arange(T, device="cuda")
    step_of_slot = T - 1 - (head - slot) % T
    k_ring = inp.k.view(1, 8, T, C, 128)[:, :, step_of_slot].reshape(1, 8, T * C, 128).contiguous()
    v_ring = inp.v.view(1, 8, T, C, 128)[:, :, step_of_slot].reshape(1, 8, T * C, 128).contiguous()
    ring, _ = mvpa_hip.mvpa_forward(q_last, k_ring, v_ring, *tabs, return_lse=True, last_step_only=True,
                                    ring_head=torch.tensor([head], dtype=torch.int32, device="cuda"))
    assert (ring.float() - ref).abs().max().item() <= 2e-2
    assert ((ring.float() - ref).norm() / ref.norm()).item() <= 5e-3


@pytest.mark.parametrize("kern", ["KERNEL_AUTO", "KERNEL_MFMA"])
def test_bf16_base_attention_shape_full_size(kern):
    """The base model's attention at full length (B1 H16 Hkv8 C128 T512 Dh128) on the build the
    library picks for it (output columns split over two waves) and on the general kernel (one
    wave on four key tiles): sampled query rows of one head against the oracle - the first
    steps, a step whose keys are mostly far, the last step - and masks through bit-exact
    perturbation, as for the irregular-channel configuration."""
    kern = getattr(mvpa_hip, kern)
    C, T = 128, 512
    inp = make_mvpa_inputs(B=1, C=C, T=T, H=16, Hkv=8, Dh=128, seed=0, qkv_unit=True,
                           validity=True).round_to(torch.bfloat16)
    d = inp.to("cuda", torch.bfloat16)
    out = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                                chan_valid=d.chan_valid, kernel=kern)
    ranges = [(0, 2 * C), (300 * C, 301 * C), (511 * C, 512 * C)]
    ref = _oracle(inp, dtype=torch.float32, heads=[(0, 11)], q_ranges=ranges, q_block=128)
    live = inp.chan_valid[0][:, None]
    for (r0, r1) in ranges:
        got = out[0, 11, r0:r1].float().cpu().view(-1, C, 128) * live
        _check_bf16(got, ref[0, 11, r0:r1].view(-1, C, 128) * live)
    dead = (~d.chan_valid)[:, None, None, :, None]
    seven = torch.tensor(7.0, dtype=torch.bfloat16, device="cuda")
    big = torch.tensor(-3.0e4, dtype=torch.bfloat16, device="cuda")
    k2 = torch.where(dead, seven, d.k.view(1, 8, T, C, 128)).view(1, 8, T * C, 128).clone()
    v2 = torch.where(dead, big, d.v.view(1, 8, T, C, 128)).view(1, 8, T * C, 128).clone()
    k2[:, :, -40 * C:] *= -1.5                        # the last 40 steps: hidden from every earlier row
    v2[:, :, -40 * C:] += 1.0
    o2 = mvpa_hip.mvpa_forward(d.q, k2, v2, d.u, d.vb, d.z, d.k_time, d.k_chan, chan_valid=d.chan_valid, kernel=kern)
    assert torch.equal(o2[:, :, :-40 * C], out[:, :, :-40 * C])
    # keys of step 0 changed: only rows with tq <= 10 and the last step keep the content term there
    k3 = d.k.clone()
    k3[:, :, :C] += 1.0
    o3 = mvpa_hip.mvpa_forward(d.q, k3, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan, chan_valid=d.chan_valid, kernel=kern)
    same = (o3 == out).flatten(0, 1).all(-1).view(-1, T, C).all(0).all(-1).cpu()
    assert same.tolist() == [not (t <= 10 or t == T - 1) for t in range(T)]
    # the fp8 content term at this length (far steps, 512 time-bias rows): the same sampled rows
    # against the oracle within the stated fp8 tolerance, and the masks bit for bit
    o8 = mvpa_hip.mvpa_forward(d.q, d.k, d.v, d.u, d.vb, d.z, d.k_time, d.k_chan,
                               chan_valid=d.chan_valid, kernel=kern, fp8_qk=True)
    assert not torch.equal(o8, out)
    tol = FP8_TOL[True]
    for (r0, r1) in ranges:
        got = o8[0, 11, r0:r1].float().cpu().view(-1, C, 128) * live
        want = ref[0, 11, r0:r1].view(-1, C, 128) * live
        err, rel = (got - want).abs().max().item(), _rel_l2(got, want)
        assert err <= tol["max_abs"] and rel <= tol["rel_l2"], f"fp8 rows {r0}: max-abs {err:.3e}, rel-L2 {rel:.3e}"
    # (values only: the keys enter the per-head fp8 scales, which are computed over every row)
    o82 = mvpa_hip.mvpa_forward(d.q, d.k, v2, d.u, d.vb, d.z, d.k_time, d.k_chan, chan_valid=d.chan_valid,
                                kernel=kern, fp8_qk=True)
    assert torch.equal(o82[:, :, :-40 * C], o8[:, :, :-40 * C])
