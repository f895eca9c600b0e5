"""Host-only checks of the C ABI: the library loads, exports every symbol the header
declares, and rejects bad argument blocks with the documented status codes.  No kernel is
launched here."""
import ctypes
import os
import re

import pytest
import torch

import mvpa_hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "mvpa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mvpa_[a-z0-9_]+)\s*\(", text)))


def test_exports_every_declared_symbol(lib):
    names = _declared_functions()
    assert "mvpa_forward" in names and "mvpa_linear_bf16" in names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mvpa_hip.h but not exported"
    assert lib.mvpa_version() == 3


def _args(B=2, H=4, Hkv=4, T=4, C=3, Dh=32, dtype=torch.float32, **kw):
    N = T * C
    q = torch.zeros((B, H, N, Dh), dtype=dtype)
    k = torch.zeros((B, Hkv, N, Dh), dtype=dtype)
    tab = torch.zeros((Hkv, max(T, C), Dh), dtype=dtype)
    return mvpa_hip.make_args(q, k, k, q, tab, tab, tab, tab, tab, T=T, C=C, sm_scale=0.1, **kw), (q, k, tab)


def test_validate_accepts_good_block(lib):
    a, keep = _args()
    assert lib.mvpa_validate(ctypes.byref(a)) == 0
    assert lib.mvpa_select_kernel(ctypes.byref(a)) == mvpa_hip.KERNEL_GENERIC   # fp32 -> generic


@pytest.mark.parametrize("mutate,code", [
    (lambda a: setattr(a, "Dh", 48), -2),
    (lambda a: setattr(a, "Hkv", 3), -3),
    (lambda a: setattr(a, "T", 0), -4),
    (lambda a: setattr(a, "C", -1), -4),
    (lambda a: setattr(a, "B", 0), -5),
    (lambda a: setattr(a, "dtype", 7), -6),
    (lambda a: setattr(a, "q", None), -1),
    (lambda a: setattr(a, "k_chan", None), -1),
    (lambda a: setattr(a, "struct_size", 8), -9),
    (lambda a: setattr(a, "flags", 2 | 4), -11),
    (lambda a: setattr(a, "q_stride_n", 8), -5),
])
def test_validate_rejects(lib, mutate, code):
    a, keep = _args()
    mutate(a)
    assert lib.mvpa_validate(ctypes.byref(a)) == code
    assert lib.mvpa_forward(ctypes.byref(a), None) == code      # rejected before any launch
    assert len(lib.mvpa_error_string(code)) > 3


def test_validate_key_split_arguments(lib):
    """n_split cuts the key steps of a MVPA_FLAG_LAST_STEP launch into runs: it needs that flag, a
    16-byte aligned workspace of mvpa_split_ws_bytes and no empty run."""
    a, keep = _args(T=6)
    assert lib.mvpa_split_ws_bytes(ctypes.byref(a)) == 0
    a.n_split = 3
    assert lib.mvpa_split_ws_bytes(ctypes.byref(a)) == 3 * 2 * 4 * 3 * (32 * 2 + 4)
    assert lib.mvpa_validate(ctypes.byref(a)) == -8              # not a last-step launch
    a.flags |= mvpa_hip.FLAG_LAST_STEP
    assert lib.mvpa_validate(ctypes.byref(a)) == -1              # no workspace
    buf = ctypes.create_string_buffer(64)
    p16 = (ctypes.addressof(buf) + 15) & ~15
    a.split_ws = p16 + 4
    assert lib.mvpa_validate(ctypes.byref(a)) == -7
    a.split_ws = p16
    assert lib.mvpa_validate(ctypes.byref(a)) == 0
    a.n_split = 4                                                # runs of 2: the fourth is empty
    assert lib.mvpa_validate(ctypes.byref(a)) == -5
    a.n_split = 7                                                # more runs than key steps
    assert lib.mvpa_validate(ctypes.byref(a)) == -5
    a.n_split = -1
    assert lib.mvpa_validate(ctypes.byref(a)) == -5
    assert mvpa_hip.default_key_splits(1, 16, 512) == 16
    assert mvpa_hip.default_key_splits(8, 64, 512) == 1
    for T in range(1, 200):                                      # never an empty run
        n = mvpa_hip.default_key_splits(1, 2, T)
        assert n >= 1 and (n - 1) * ((T + n - 1) // n) < T


def test_wide_row_pitch_leaves_the_matrix_core_kernels(lib):
    """The matrix-core kernels keep the offsets of q and o rows of a sample in 32 bits: a view whose
    row pitch makes them wrap must not be taken by them (AUTO falls back to the row-per-lane
    kernel, a forced matrix-core selector is refused).  Host-side only: nothing is launched."""
    a, keep = _args(B=1, H=2, Hkv=2, T=64, C=64, Dh=64, dtype=torch.bfloat16)
    assert lib.mvpa_select_kernel(ctypes.byref(a)) == mvpa_hip.KERNEL_MFMA
    for field in ("q_stride_n", "o_stride_n", "k_stride_n", "v_stride_n"):
        a, keep = _args(B=1, H=2, Hkv=2, T=64, C=64, Dh=64, dtype=torch.bfloat16)
        setattr(a, field, 1 << 20)                              # 4096 rows x 2^20 elements
        assert lib.mvpa_select_kernel(ctypes.byref(a)) == mvpa_hip.KERNEL_GENERIC, field
        for forced in (mvpa_hip.KERNEL_MFMA, mvpa_hip.KERNEL_MFMA_STEP, mvpa_hip.KERNEL_MFMA_SPLIT):
            a.kernel = forced
            assert lib.mvpa_validate(ctypes.byref(a)) == -8, field
    # the pitch of a fused projection output at the largest benchmark shape stays inside
    a, keep = _args(B=1, H=2, Hkv=2, T=64, C=64, Dh=64, dtype=torch.bfloat16)
    a.T, a.C, a.q_stride_n, a.o_stride_n = 512, 128, 4096, 2048
    a.k_stride_n = a.v_stride_n = 4096
    assert lib.mvpa_select_kernel(ctypes.byref(a)) == mvpa_hip.KERNEL_MFMA


@pytest.mark.parametrize("B,H,Hkv,nt", [(4, 16, 16, 33), (4, 12, 4, 33), (1, 16, 8, 512), (8, 16, 16, 128),
                                        (2, 8, 2, 5), (3, 5, 5, 7), (1, 4, 1, 9), (2, 16, 4, 1), (1, 16, 8, 2)])
def test_block_order_is_a_permutation_and_keeps_kv_groups_on_one_xcd(lib, B, H, Hkv, nt):
    """Every (pair, tile) is handed out exactly once; the last tile of every pair goes out first;
    and where the pairs divide over the 8 XCDs, the heads of a kv group share an XCD whenever an
    XCD's share of heads is a whole number of groups."""
    import numpy as np
    nbh, grp = B * H, H // Hkv
    bh = np.full(nbh * nt, -1, dtype=np.int32)
    tile = np.full(nbh * nt, -1, dtype=np.int32)
    assert lib.mvpa_debug_block_order(nbh, nt, grp, bh.ctypes.data, tile.ctypes.data) == 0
    seen = set(zip(bh.tolist(), tile.tolist()))
    assert len(seen) == nbh * nt and min(bh) == 0 and max(bh) == nbh - 1 and min(tile) == 0 and max(tile) == nt - 1
    if nt > 1:
        assert set(tile[:nbh].tolist()) == {nt - 1} and (nt - 1) not in set(tile[nbh:].tolist())
    if nbh % 8 == 0 and nt > 1:
        xcd = np.arange(nbh * nt) % 8
        owner = {}
        for x, p in zip(xcd.tolist(), bh.tolist()):
            assert owner.setdefault(p, x) == x, "a (b, h) pair is split over two XCDs"
        if (nbh // 8) % grp == 0:
            for p, x in owner.items():
                assert owner[(p // grp) * grp] == x, "a kv group is split over two XCDs"
            # within a group the heads take a tile side by side
            first = nbh + int(np.argmax(xcd[nbh:] == 0))
            if grp > 1:
                run = [(int(bh[first + 8 * i]), int(tile[first + 8 * i])) for i in range(grp * (2 if nbh // 8 // grp == 2 else 1))]   # two units: interleaved
                mine = [(p, t) for p, t in run if p // grp == run[0][0] // grp]
                assert len({p for p, _ in mine}) == grp and len({t for _, t in mine}) == 1


def test_new_entry_points_reject_bad_arguments(lib):
    """Host-side validation of the entry points around the fp8 content term, the fp32 product and
    the norm-in-the-products path: every rejection comes back before anything is launched."""
    buf = ctypes.create_string_buffer(256)
    p16 = (ctypes.addressof(buf) + 15) & ~15
    assert lib.mvpa_linear_f32(None, None, None, 1, 1, 1, 1, 1, 1, None) == -1
    assert lib.mvpa_linear_f32(p16, p16, p16, 4, 4, 8, 4, 8, 4, None) == -5              # ldx < K
    assert lib.mvpa_row_sumsq_bf16(None, None, 1, 8, 8, None) == -1
    assert lib.mvpa_row_sumsq_bf16(p16, p16, 4, 12, 16, None) == -7                      # cols not a multiple of 8
    assert lib.mvpa_row_sumsq_bf16(p16, p16, 4, 16, 8, None) == -5                       # ldx < cols
    assert lib.mvpa_linear_sumsq_parts(16384, 768) == 8 and lib.mvpa_linear_sumsq_parts(65536, 2048) == 16
    assert lib.mvpa_linear_sumsq_parts(0, 8) == 0
    assert lib.mvpa_linear_bf16_residual_sumsq(p16, p16, p16, p16, None, 512, 64, 128, 128, 128, 64, 64, None) == -1
    assert lib.mvpa_linear_bf16_residual_sumsq(p16, p16, p16, p16, p16, 512, 60, 128, 128, 128, 64, 64, None) == -7   # N % 8
    assert lib.mvpa_linear_bf16_residual_sumsq(p16, p16, p16, p16, p16, 64, 64, 128, 128, 128, 64, 64, None) == -8    # too few rows
    assert lib.mvpa_linear_bf16_dual_normed(p16, p16, p16, p16, p16, 512, 64, 64, 128, 128, 128, 64, 128, 64,
                                            None, 8, 1e-5, None) == -1
    assert lib.mvpa_linear_bf16_dual_normed(p16, p16, p16, p16, p16, 512, 64, 64, 128, 128, 128, 64, 128, 64,
                                            p16, 0, 1e-5, None) == -5
    a, keep = _args(B=1, H=2, Hkv=2, T=8, C=40, Dh=64, dtype=torch.bfloat16)
    assert lib.mvpa_fp8_prepare(None, p16, p16, None, None) == -1
    assert lib.mvpa_fp8_prepare(ctypes.byref(a), None, p16, None, None) == -1
    a.struct_size = 16
    assert lib.mvpa_fp8_prepare(ctypes.byref(a), p16, p16, None, None) == -9
    a, keep = _args(B=1, H=2, Hkv=2, T=8, C=40, Dh=64, dtype=torch.float32)
    assert lib.mvpa_fp8_prepare(ctypes.byref(a), p16, p16, None, None) == -8             # bf16 only
    a, keep = _args(B=1, H=3, Hkv=2, T=8, C=40, Dh=64, dtype=torch.bfloat16)
    assert lib.mvpa_fp8_prepare(ctypes.byref(a), p16, p16, None, None) == -3
    # the column-split build needs the keys' e4m3 copy for the fp8 content term
    a, keep = _args(B=1, H=2, Hkv=2, T=8, C=100, Dh=128, dtype=torch.bfloat16)
    a.flags |= mvpa_hip.FLAG_FP8_QK
    a.fp8_q_scale = a.fp8_k_scale = p16
    a.kernel = mvpa_hip.KERNEL_MFMA_SPLIT
    assert lib.mvpa_validate(ctypes.byref(a)) == -8
    a.k_fp8 = p16
    assert lib.mvpa_validate(ctypes.byref(a)) == 0
    a.kernel = mvpa_hip.KERNEL_AUTO
    a.k_fp8 = None
    assert lib.mvpa_validate(ctypes.byref(a)) == 0          # AUTO then keeps the general kernel


def test_null_block(lib):
    assert lib.mvpa_validate(None) == -1


def test_dense_entry_points_reject_bad_arguments(lib):
    assert lib.mvpa_linear_bf16(None, None, None, 1, 1, 1, 1, 1, 1, 0, None) == -1
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    assert lib.mvpa_linear_bf16(p16, p16, p16, 4, 4, 8, 4, 8, 4, 0, None) == -5   # ldx < K
    assert lib.mvpa_linear_bf16(p16 + 2, p16, p16, 4, 4, 8, 8, 8, 4, 0, None) == -7
    assert lib.mvpa_linear_bf16_residual(None, None, None, None, 1, 1, 1, 1, 1, 1, 1, None) == -1
    assert lib.mvpa_linear_bf16_residual(p16, p16, p16, p16, 4, 4, 8, 8, 8, 2, 4, None) == -5     # ldr < N
    assert lib.mvpa_linear_bf16_residual(p16, p16, p16, p16, 4, 4, 8, 8, 8, 4, 4, None) < 0        # too small for the tiled kernel
    assert lib.mvpa_linear_bf16_dual(None, None, None, None, None, 1, 1, 1, 1, 1, 1, 1, 1, 1, None) == -1
    assert lib.mvpa_linear_bf16_dual(p16, p16, p16, p16, p16, 4, 4, 4, 8, 8, 8, 2, 8, 4, None) == -5   # ldy0 < N0
    assert lib.mvpa_linear_bf16_dual(p16, p16, p16, p16, p16, 4, 4, 4, 8, 8, 8, 4, 8, 4, None) < 0      # too small
    assert lib.mvpa_cosine_rows_bf16(None, None, None, 1, 1, 8, 8, 8, 8, 8, 1e-8, None) == -1
    assert lib.mvpa_cosine_rows_bf16(p16, p16, p16, 1, 1, 12, 16, 16, 16, 16, 1e-8, None) == -7   # cols not a multiple of 8
    assert lib.mvpa_rmsnorm(None, None, None, 1, 1, 1, 1, 1e-5, 0, 0, None) == -1
    assert lib.mvpa_wavedec_db4(p16, p16, 1, 512, 6, 549, 549, None) == -5       # wrong dwt_size
    assert lib.mvpa_debug_maps(0, 3, 10, 15, None, p16, p16, p16, None) == -4


def test_python_operator_errors():
    """Same exception types as the reference operator (attentions/attn.py:1041-1045, 1339, 1344)."""
    from attentions import flashmvpa
    q = torch.zeros(1, 4, 12, 32)
    kv = torch.zeros(1, 3, 12, 32)
    b = torch.zeros(1, 3, 1, 32)
    with pytest.raises(AssertionError):
        flashmvpa(q, b, b, b, kv, torch.zeros(1, 3, 4, 32), torch.zeros(1, 3, 3, 32), kv, True, 0.1)
    kv = torch.zeros(1, 4, 12, 32)
    b = torch.zeros(1, 4, 1, 32)
    with pytest.raises(AssertionError):      # N != T*C
        flashmvpa(q, b, b, b, kv, torch.zeros(1, 4, 5, 32), torch.zeros(1, 4, 3, 32), kv, True, 0.1)
    with pytest.raises(NotImplementedError):  # a content window without the relative biases
        flashmvpa(q, b, b, b, kv, torch.zeros(1, 4, 4, 32), torch.zeros(1, 4, 3, 32), kv, False, 0.1,
                  window_size=10, rel_bias_time=False, rel_bias_chan=False)
    with pytest.raises(RuntimeError):        # CPU tensors: no fallback path, with dropout neither
        flashmvpa(q, b, b, b, kv, torch.zeros(1, 4, 4, 32), torch.zeros(1, 4, 3, 32), kv, True, 0.1,
                  p_drop=0.1)
    with pytest.raises(RuntimeError):        # CPU tensors: no fallback path
        flashmvpa(q, b, b, b, kv, torch.zeros(1, 4, 4, 32), torch.zeros(1, 4, 3, 32), kv, True, 0.1)


def test_layer_state_dict_names():
    from types import SimpleNamespace
    from layers import MVPFormerGQAAttention, MVPFormerGQAFlashAttention
    cfg = SimpleNamespace(max_position_embeddings=16, hidden_size=64, num_attention_heads=4,
                          n_head_kv=2, n_inner=128, global_att=True, scale_attn_weights=True,
                          scale_attn_by_inverse_layer_idx=False, reorder_and_upcast_attn=False,
                          lora=False, attn_pdrop=0.1, resid_pdrop=0.1)
    for cls in (MVPFormerGQAAttention, MVPFormerGQAFlashAttention):
        m = cls(cfg, layer_idx=0)
        assert sorted(m.state_dict().keys()) == sorted([
            "q_attn.weight", "c_attn.weight", "position_net.weight", "channel_net.weight",
            "c_proj.weight", "attn_bias", "time_bias", "masked_bias"])
        assert m.c_attn.weight.shape == (2 * 32, 64) and m.attn_bias.shape == (3 * 32,)
    cfg.lora, cfg.lora_rank, cfg.lora_alpha, cfg.lora_dropout, cfg.lora_merge = True, 8, 16, 0, True
    m = MVPFormerGQAAttention(cfg)
    keys = m.state_dict().keys()
    for n in m.adapter_params():
        assert n in keys
    assert m.c_attn.lora_B.shape == (32, 8) and m.q_attn.lora_A.shape == (8, 64)
    cfg.hidden_size = 66
    with pytest.raises(ValueError):
        MVPFormerGQAAttention(cfg)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: with --gpus above 1 (or under a multi-rank launcher) it exits
    with a message that says so, before touching any device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert res.returncode == 2
    assert "ONE GPU" in res.stderr and res.stdout.strip() == ""
    env = dict(os.environ, WORLD_SIZE="2")
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py")], capture_output=True,
                         text=True, timeout=120, env=env)
    assert res.returncode == 2 and "ONE GPU" in res.stderr


def test_kv_cache_window_logic_on_the_host():
    """MvpaKVCache is plain tensor bookkeeping: appending past max_steps keeps exactly the last
    max_steps time steps, in order, through every wrap of the buffer (runs on the CPU)."""
    from layers import MvpaKVCache
    for max_steps, slack in ((5, 2), (4, 0), (1, 3), (7, None)):
        cache = MvpaKVCache(1, 2, 3, 4, max_steps=max_steps, dtype=torch.float32, device="cpu", slack=slack)
        assert cache.capacity >= max_steps
        for i in range(4 * cache.capacity + 3):
            k, v = cache.append(torch.full((1, 2, 3, 4), float(i)), torch.full((1, 2, 3, 4), -float(i)))
            want = torch.arange(max(0, i - max_steps + 1), i + 1, dtype=torch.float32)
            assert k.shape == (1, 2, len(want), 3, 4)
            assert torch.equal(k[0, 1, :, 2, 3], want) and torch.equal(v[0, 0, :, 0, 0], -want)
            assert cache.start + cache.length <= cache.capacity
        cache.reset()
        assert cache.length == 0
    with pytest.raises(ValueError):
        MvpaKVCache(1, 1, 1, 8, max_steps=0, device="cpu")
