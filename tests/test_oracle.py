"""Pins the CPU oracle (oracle/mvpa_oracle.py) without the GPU: closed-form index maps,
a library special case (torch SDPA), a float64 brute force, and invariants chosen so that a
dropped term, a wrong sign or index, or a transposed operand fails at least one of them."""
import math

import pytest
import torch

from mvpa_hip.synthetic import make_mvpa_inputs
from oracle import mvpa_oracle as O


def _five_d(inp):
    B, H, N, Dh = inp.q.shape
    Hkv = inp.k.shape[1]
    T, C = inp.T, inp.C
    q = inp.q.view(B, H, T, C, Dh)
    k = inp.k.view(B, Hkv, T, C, Dh)
    v = inp.v.view(B, Hkv, T, C, Dh)
    tk = inp.k_time.view(1, Hkv, T, 1, Dh)
    ck = inp.k_chan.view(1, Hkv, 1, C, Dh)
    bias = torch.cat([inp.u.reshape(-1), inp.vb.reshape(-1), inp.z.reshape(-1)])
    return q, k, tk, ck, v, bias


def _rel_attn(inp, **kw):
    q, k, tk, ck, v, bias = _five_d(inp)
    out, w = O.rel_attn(q, k, tk, ck, v, bias, **kw)
    return out.flatten(2, 3), w


@pytest.mark.parametrize("T,C", [(5, 3), (7, 1), (4, 8), (12, 5)])
def test_rel_shift_closed_form(T, C):
    """Iota-coded table: x[n, j] = n*T + j.  After the shift column tk must hold
    x[n, T-1-(tq-tk)] for every tk <= tq (bit exact)."""
    N = T * C
    x = torch.arange(N * T, dtype=torch.float32).view(1, 1, N, T)
    y = O.rel_shift(x)
    for n in range(N):
        tq = n // C
        for tk in range(tq + 1):
            assert y[0, 0, n, tk].item() == n * T + (T - 1 - (tq - tk))


@pytest.mark.parametrize("T,C", [(3, 1), (2, 2), (3, 5), (2, 9)])
def test_rel_shift_chan_closed_form(T, C):
    N = T * C
    x = torch.arange(N * C, dtype=torch.float32).view(1, 1, N, C)
    y = O.rel_shift_chan(x)
    for n in range(N):
        cq = n % C
        for ck in range(C):
            assert y[0, 0, n, ck].item() == n * C + (C - 1 - abs(cq - ck))


def test_repeat_helpers_layout():
    x = torch.arange(6.0).view(1, 1, 2, 3)
    assert O.repeat_channel(x, 2)[0, 0, 0].tolist() == [0, 0, 1, 1, 2, 2]
    assert O.repeat_time(x, 2)[0, 0, 1].tolist() == [3, 4, 5, 3, 4, 5]


def test_rel_attn_matches_sdpa_when_window_vacuous():
    """T <= 11 makes the content window all-ones, so MVPA is ordinary attention with an
    additive bias: torch's scaled_dot_product_attention pins the whole op."""
    inp = make_mvpa_inputs(B=2, C=4, T=9, H=4, Dh=16, Hkv=2, seed=3, table_std=0.5)
    out, _ = _rel_attn(inp)
    B, H, N, Dh = inp.q.shape
    T, C, grp = inp.T, inp.C, 2
    n = torch.arange(N)
    tq, cq = (n // C)[:, None], (n % C)[:, None]
    tk, ck = (n // C)[None, :], (n % C)[None, :]
    s = 1 / math.sqrt(Dh)
    u = inp.u.repeat_interleave(grp, 0)
    vb = inp.vb.repeat_interleave(grp, 0)
    z = inp.z.repeat_interleave(grp, 0)
    r = inp.k_time.repeat_interleave(grp, 0)
    e = inp.k_chan.repeat_interleave(grp, 0)
    st = torch.einsum("bhnd,htd->bhnt", inp.q + vb[None, :, None], r)
    sc = torch.einsum("bhnd,hcd->bhnc", inp.q + z[None, :, None], e)
    ti = (T - 1 - (tq - tk)).clamp(0, T - 1).expand(B, H, N, N)
    ci = (C - 1 - (cq - ck).abs()).expand(B, H, N, N)
    bias = (torch.gather(st, 3, ti) + torch.gather(sc, 3, ci)) * s
    bias = bias.masked_fill((tk > tq)[None, None], float("-inf"))
    ref = torch.nn.functional.scaled_dot_product_attention(
        inp.q + u[None, :, None], inp.k.repeat_interleave(grp, 1), inp.v.repeat_interleave(grp, 1),
        attn_mask=bias, scale=s)
    assert torch.allclose(out, ref, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("window,global_att", [(10, True), (2, True), (10, False)])
def test_rel_attn_matches_bruteforce(window, global_att):
    """Windowed case (T > window+1) against float64 loops from the definition, with GQA."""
    inp = make_mvpa_inputs(B=1, C=3, T=13, H=2, Dh=4, Hkv=1, seed=5, table_std=0.7)
    out, _ = _rel_attn(inp, window=window, global_att=global_att)
    ref = O.mvpa_bruteforce(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                            window=window, global_att=global_att)
    assert (out.double() - ref).abs().max().item() < 5e-6


def test_direct_matches_bruteforce_with_validity():
    inp = make_mvpa_inputs(B=2, C=4, T=12, H=2, Dh=4, Hkv=2, seed=8, table_std=0.7, validity=True)
    inp.chan_valid[0, 1] = False
    out = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                        chan_valid=inp.chan_valid)
    ref = O.mvpa_bruteforce(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                            chan_valid=inp.chan_valid)
    assert (out - ref).abs().max().item() < 1e-12


@pytest.mark.parametrize("cfg", [dict(B=2, C=8, T=32, H=4, Dh=32), dict(B=1, C=5, T=14, H=4, Dh=16, Hkv=2)])
def test_direct_matches_rel_attn(cfg):
    """The chunked closed form equals the op-by-op restatement, also for config c1's shape and
    with the channel validity expressed as the reference's additive attention_mask."""
    inp = make_mvpa_inputs(seed=0, validity=True, table_std=0.3, **cfg)
    B, H, N, Dh = inp.q.shape
    am = (~inp.chan_valid).float()[:, None, :].expand(B, inp.T, inp.C).reshape(B, 1, 1, N)
    am = am * torch.finfo(torch.float32).min
    out, w = _rel_attn(inp, attention_mask=am)
    direct, lse = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                                chan_valid=inp.chan_valid, q_block=64, return_lse=True)
    assert (out.double() - direct).abs().max().item() < 5e-6
    # masked keys carry exactly zero weight
    C = inp.C
    dead = (~inp.chan_valid)[:, None, None, :].expand(B, H, N, C).repeat(1, 1, 1, inp.T)
    assert (w[dead] == 0).all()


def test_invariants():
    inp = make_mvpa_inputs(B=1, C=3, T=16, H=2, Dh=8, seed=11, table_std=0.5)
    T, C = inp.T, inp.C

    def run(i):
        return _rel_attn(i)[0]

    base = run(inp)
    # rows are probability-weighted averages: V == 1 gives exactly ~1
    ones = make_mvpa_inputs(B=1, C=3, T=16, H=2, Dh=8, seed=11, table_std=0.5)
    ones.v = torch.ones_like(ones.v)
    assert torch.allclose(run(ones), torch.ones_like(base), atol=1e-6)
    # causality: changing K and V at the last time step leaves earlier rows unchanged
    pert = make_mvpa_inputs(B=1, C=3, T=16, H=2, Dh=8, seed=11, table_std=0.5)
    pert.k[:, :, -C:] += 3.0
    pert.v[:, :, -C:] -= 2.0
    assert torch.equal(run(pert)[:, :, :-C], base[:, :, :-C])
    # window locality: K at time 0 matters only to tq <= 10 and to the last time step
    pert = make_mvpa_inputs(B=1, C=3, T=16, H=2, Dh=8, seed=11, table_std=0.5)
    pert.k[:, :, :C] += 1.0
    out = run(pert)
    changed = (out != base).flatten(0, 1).any(-1).view(-1, T, C).any(0).any(-1)
    expect = torch.tensor([t <= 10 or t == T - 1 for t in range(T)])
    assert torch.equal(changed, expect)
    # GQA == MHA with replicated kv heads, tables and biases
    g = make_mvpa_inputs(B=1, C=3, T=16, H=4, Dh=8, Hkv=2, seed=12, table_std=0.5)
    full = make_mvpa_inputs(B=1, C=3, T=16, H=4, Dh=8, Hkv=2, seed=12, table_std=0.5)
    for name in ("k", "v"):
        setattr(full, name, getattr(g, name).repeat_interleave(2, 1))
    for name in ("k_time", "k_chan", "u", "vb", "z"):
        setattr(full, name, getattr(g, name).repeat_interleave(2, 0))
    assert torch.allclose(run(g), run(full), atol=1e-6)


def test_scale_flags():
    inp = make_mvpa_inputs(B=1, C=2, T=6, H=2, Dh=8, seed=2, table_std=0.5)
    a = _rel_attn(inp, scale_attn_by_inverse_layer_idx=True, layer_idx=2)[0]
    b = O.mvpa_direct(inp.q, inp.k, inp.v, inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan,
                      sm_scale=1 / math.sqrt(8) / 3.0)
    assert (a.double() - b).abs().max().item() < 5e-6


def test_db4_filter_bank_properties():
    lo = torch.tensor(O.DB4_DEC_LO, dtype=torch.float64)
    hi = torch.tensor(O.DB4_DEC_HI, dtype=torch.float64)
    assert abs(lo.sum().item() - math.sqrt(2)) < 1e-12
    assert abs((lo * lo).sum().item() - 1) < 1e-12
    for sh in (2, 4, 6):
        assert abs((lo[sh:] * lo[:-sh]).sum().item()) < 1e-12
    assert abs((lo * hi).sum().item()) < 1e-12
    k = torch.arange(8, dtype=torch.float64)
    for p in range(4):                      # four vanishing moments of the high-pass filter
        assert abs((hi * k ** p).sum().item()) < 1e-9
    assert O.dwt_sizes(512) == [259, 133, 70, 38, 22, 14, 14] and sum(O.dwt_sizes(512)) == 550
    assert sum(O.dwt_sizes(2560)) == 2610
    # even length, periodic extension: the level is an orthogonal map on the first n/2 outputs
    x = torch.randn(3, 64, dtype=torch.float64)
    a, d = O.dwt_level_periodic(x)
    n2 = 32
    # outputs k >= n/2 repeat outputs k - n/2 (periodicity of the extension)
    assert torch.allclose(a[:, n2:], a[:, : a.shape[1] - n2]) and torch.allclose(d[:, n2:], d[:, : d.shape[1] - n2])
    energy = (a[:, :n2] ** 2).sum(-1) + (d[:, :n2] ** 2).sum(-1)
    assert torch.allclose(energy, (x ** 2).sum(-1))


def _wavedec_pad_conv(x):
    """Second, independent statement of what the reference's encoder asks its wavelet library for
    (models/fftencoder.py:80-88: ptwt.wavedec(x, db4, mode="periodic"), outputs concatenated).
    The library's published algorithm, level by level: pad the signal circularly by
    (2*8 - 3) // 2 = 6 samples on the left and 6 (+1 if the length is odd) on the right, then one
    stride-2 conv1d (cross-correlation) with the FLIPPED decomposition filters [dec_lo, dec_hi];
    the approximation goes on to the next level, floor(log2(n / 7)) levels in all; the result is
    [cA_L, cD_L, ..., cD_1].  Written with torch's pad and conv1d, not with the index formula the
    oracle uses."""
    F = torch.nn.functional
    lo = torch.tensor(O.DB4_DEC_LO, dtype=x.dtype).flip(0)
    hi = torch.tensor(O.DB4_DEC_HI, dtype=x.dtype).flip(0)
    filt = torch.stack([lo, hi])[:, None, :]                  # [2, 1, 8]
    a = x[:, None, :]
    details = []
    levels = int(math.floor(math.log2(x.shape[-1] / 7)))
    for _ in range(levels):
        n = a.shape[-1]
        padded = F.pad(a, (6, 6 + n % 2), mode="circular")
        res = F.conv1d(padded, filt, stride=2)                # [M, 2, floor((n + 7) / 2)]
        a, d = res[:, :1], res[:, 1]
        details.append(d)
    return torch.cat([a[:, 0]] + details[::-1], dim=-1)


@pytest.mark.parametrize("L", [512, 2560, 97, 333, 1001])
def test_wavedec_matches_pad_and_conv1d_statement(L):
    """Pins wavedec_db4_periodic: equal to the pad + strided-conv1d statement of the wavelet
    library's algorithm for the shipped segment lengths (512 in the benchmark configurations, 2560
    in the YAMLs) and for odd lengths, where the right pad grows by one; sizes as
    models/fftencoder.py:70-78 computes them."""
    x = torch.randn(5, L, dtype=torch.float64, generator=torch.Generator().manual_seed(L))
    want = _wavedec_pad_conv(x)
    got = O.wavedec_db4_periodic(x.float())
    assert got.shape == want.shape and got.shape[-1] == sum(O.dwt_sizes(L))
    assert (got.double() - want).abs().max().item() <= 2e-5
    # one level, float64 against float64: the same numbers to rounding of the summation order
    a, d = O.dwt_level_periodic(x)
    F = torch.nn.functional
    padded = F.pad(x[:, None], (6, 6 + L % 2), mode="circular")
    lo = torch.tensor(O.DB4_DEC_LO, dtype=torch.float64).flip(0)[None, None]
    hi = torch.tensor(O.DB4_DEC_HI, dtype=torch.float64).flip(0)[None, None]
    assert torch.allclose(a, F.conv1d(padded, lo, stride=2)[:, 0], atol=1e-13)
    assert torch.allclose(d, F.conv1d(padded, hi, stride=2)[:, 0], atol=1e-13)


def test_wavedec_phase_on_unit_impulses():
    """The phase (alignment) convention, spelled out on unit impulses by hand from the pad + conv1d
    definition: with 6 samples of left pad and the flipped filter, output k of a level reads the
    padded samples 2k .. 2k+7, i.e. signal samples 2k-6 .. 2k+1, against dec_lo[7] .. dec_lo[0].
    An impulse at sample p therefore puts dec_lo[2k+1-p] into approximation coefficient k."""
    lo, hi = O.DB4_DEC_LO, O.DB4_DEC_HI
    n = 16                                        # one level at this length (floor(log2(16/7)) = 1)
    for p, taps in ((0, {0: 1, 1: 3, 2: 5, 3: 7, 8: 1, 9: 3, 10: 5}),       # k: index into dec_lo
                    (5, {2: 0, 3: 2, 4: 4, 5: 6, 10: 0}),
                    (15, {0: 2, 1: 4, 2: 6, 7: 0, 8: 2, 9: 4, 10: 6})):
        x = torch.zeros(1, n)
        x[0, p] = 1.0
        out = O.wavedec_db4_periodic(x)[0]
        m = (n + 7) // 2
        assert out.shape[0] == 2 * m
        for k in range(m):
            want_a = lo[taps[k]] if k in taps else 0.0
            want_d = hi[taps[k]] if k in taps else 0.0
            assert abs(out[k].item() - want_a) < 1e-7, (p, k)
            assert abs(out[m + k].item() - want_d) < 1e-7, (p, k)


def test_golden_c1_fixture():
    """Oracle and input generator against the committed vector (tests/golden/c1_seed0.npz)."""
    import os
    import numpy as np
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "c1_seed0.npz"))
    inp = make_mvpa_inputs(B=2, C=8, T=32, H=4, Dh=32, seed=0)
    assert np.array_equal(inp.q[0, 0, :4].numpy(), g["q_probe"])
    assert np.array_equal(inp.k_time[0, :2].numpy(), g["k_time_probe"])
    out, _ = _rel_attn(inp)
    assert np.abs(out.numpy() - g["out"]).max() <= 5e-6


def test_direct_gradcheck():
    """The closed-form oracle is differentiable and its reverse-mode gradient agrees with finite
    differences (float64, windowed, GQA): the reference for the backward parity tests."""
    torch.manual_seed(0)
    B, H, Hkv, T, C, Dh = 1, 2, 1, 5, 2, 4
    mk = lambda *s: (torch.randn(*s, dtype=torch.float64) * 0.5).requires_grad_(True)  # noqa: E731
    q, k, v = mk(B, H, T * C, Dh), mk(B, Hkv, T * C, Dh), mk(B, Hkv, T * C, Dh)
    u, vb, z = mk(Hkv, Dh), mk(Hkv, Dh), mk(Hkv, Dh)
    kt, kc = mk(Hkv, T, Dh), mk(Hkv, C, Dh)
    assert torch.autograd.gradcheck(lambda *a: O.mvpa_direct(*a, window=2),
                                    (q, k, v, u, vb, z, kt, kc), eps=1e-6, atol=1e-6)
