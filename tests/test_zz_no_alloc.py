"""The decoding step on the workspace built into the library (mvpa_forward_last_step_static, for
callers that cannot allocate device memory) against the same step through mvpa_forward with a
caller-allocated workspace: the same kernels on the same operands, so bit for bit - on two calls
in a row, the second smaller, so that what the first left in the shared array is in the way."""
import ctypes

import pytest
import torch

import mvpa_hip
from mvpa_hip.synthetic import make_mvpa_inputs

pytestmark = pytest.mark.gpu


def _step(lib, cfg, n_split, seed, entry):
    """One decoding step through the C ABI; entry is 'static' or 'caller'.  Every buffer the call
    touches is allocated here, before it."""
    inp = make_mvpa_inputs(seed=seed, qkv_unit=True, **cfg).to("cuda", torch.bfloat16)
    B, C, T, H, Dh = cfg["B"], cfg["C"], cfg["T"], cfg["H"], cfg["Dh"]
    q_last = inp.q[:, :, -C:]
    valid = torch.ones(B, C, dtype=torch.uint8, device="cuda")
    valid[:, 2::7] = 0
    out = torch.full((B, H, C, Dh), float("nan"), dtype=torch.bfloat16, device="cuda")
    lse = torch.full((B, H, C), float("nan"), dtype=torch.float32, device="cuda")
    tabs = [t.contiguous() for t in (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)]
    a = mvpa_hip.make_args(q_last, inp.k, inp.v, out, *tabs, T=T, C=C, sm_scale=Dh ** -0.5,
                           flags=15 | mvpa_hip.FLAG_LAST_STEP, chan_valid=valid, lse=lse,
                           kernel=mvpa_hip.KERNEL_MFMA, n_split=n_split)
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "static":
        assert a.split_ws is None
        st = lib.mvpa_forward_last_step_static(ctypes.byref(a), stream)
    else:
        ws = torch.empty(lib.mvpa_split_ws_bytes(ctypes.byref(a)), dtype=torch.uint8, device="cuda")
        a.split_ws = ws.data_ptr()
        st = lib.mvpa_forward(ctypes.byref(a), stream)
    assert st == 0, mvpa_hip.error_string(st)
    torch.cuda.synchronize()
    return out, lse


def test_static_workspace_step_equals_caller_workspace_step():
    lib = mvpa_hip.load_library()
    big = dict(B=2, C=117, T=45, H=4, Hkv=2, Dh=64)        # keys in two parts, 4 runs
    small = dict(B=1, C=20, T=24, H=2, Hkv=1, Dh=128)      # afterwards: fewer, shorter rows
    for cfg, n, seed in ((big, 4, 51), (small, 3, 52), (big, 5, 53)):
        got, lse_got = _step(lib, cfg, n, seed, "static")
        want, lse_want = _step(lib, cfg, n, seed, "caller")
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want)
        assert torch.equal(lse_got, lse_want)


def test_static_workspace_limits():
    lib = mvpa_hip.load_library()
    assert lib.mvpa_static_ws_bytes() == 16 << 20
    cfg = dict(B=1, C=128, T=64, H=16, Hkv=8, Dh=128)
    inp = make_mvpa_inputs(seed=1, **cfg).to("cuda", torch.bfloat16)
    out = torch.empty((1, 16, 128, 128), dtype=torch.bfloat16, device="cuda")
    tabs = (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)
    a = mvpa_hip.make_args(inp.q[:, :, -128:], inp.k, inp.v, out, *tabs, T=64, C=128, sm_scale=0.1,
                           flags=15 | mvpa_hip.FLAG_LAST_STEP, kernel=mvpa_hip.KERNEL_MFMA, n_split=64)
    assert lib.mvpa_split_ws_bytes(ctypes.byref(a)) > 16 << 20
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.mvpa_forward_last_step_static(ctypes.byref(a), stream) == -12      # MVPA_ERR_WS_SIZE
    a.n_split = 1
    assert lib.mvpa_forward_last_step_static(ctypes.byref(a), stream) == -8       # nothing to split
    a.n_split, a.flags = 4, 15
    assert lib.mvpa_forward_last_step_static(ctypes.byref(a), stream) == -8       # not a decoding step
    # the binding's switch
    got = mvpa_hip.mvpa_forward(inp.q[:, :, -128:], inp.k, inp.v, *tabs, last_step_only=True,
                                key_splits=8, static_ws=True, out=out)
    want = mvpa_hip.mvpa_forward(inp.q[:, :, -128:], inp.k, inp.v, *tabs, last_step_only=True, key_splits=8)
    assert torch.equal(got, want)


def test_static_step_allocates_nothing_and_replays_in_a_graph():
    """With every buffer in place beforehand the entry point leaves the allocator's counters where
    they were, and a step recorded into a HIP graph (after mvpa_static_ws_init, so that nothing is
    looked up during capture) gives on every replay what the eager caller-workspace step gives on
    the same cache contents - replays with eager work and synchronisations between them."""
    lib = mvpa_hip.load_library()
    cfg = dict(B=2, C=64, T=40, H=4, Hkv=2, Dh=64)
    B, C, T, H, Dh = cfg["B"], cfg["C"], cfg["T"], cfg["H"], cfg["Dh"]
    inp = make_mvpa_inputs(seed=61, qkv_unit=True, **cfg).to("cuda", torch.bfloat16)
    q_last = inp.q[:, :, -C:].contiguous()
    out = torch.zeros((B, H, C, Dh), dtype=torch.bfloat16, device="cuda")
    tabs = [t.contiguous() for t in (inp.u, inp.vb, inp.z, inp.k_time, inp.k_chan)]
    a = mvpa_hip.make_args(q_last, inp.k, inp.v, out, *tabs, T=T, C=C, sm_scale=Dh ** -0.5,
                           flags=15 | mvpa_hip.FLAG_LAST_STEP, kernel=mvpa_hip.KERNEL_MFMA, n_split=5)
    assert lib.mvpa_static_ws_init() == 0
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert lib.mvpa_forward_last_step_static(ctypes.byref(a), stream) == 0
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
    eager = out.clone()

    def caller_ws_step():
        res = torch.empty_like(out)
        b = mvpa_hip.make_args(q_last, inp.k, inp.v, res, *tabs, T=T, C=C, sm_scale=Dh ** -0.5,
                               flags=15 | mvpa_hip.FLAG_LAST_STEP, kernel=mvpa_hip.KERNEL_MFMA, n_split=5)
        ws = torch.empty(lib.mvpa_split_ws_bytes(ctypes.byref(b)), dtype=torch.uint8, device="cuda")
        b.split_ws = ws.data_ptr()
        assert lib.mvpa_forward(ctypes.byref(b), torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        return res

    assert torch.equal(eager, caller_ws_step())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = lib.mvpa_forward_last_step_static(ctypes.byref(a), torch.cuda.current_stream().cuda_stream)
    assert st == 0
    for i in range(4):
        # new cache contents and a new query in the same buffers, written by eager work
        fresh = make_mvpa_inputs(seed=70 + i, qkv_unit=True, **cfg).to("cuda", torch.bfloat16)
        inp.k.copy_(fresh.k)
        inp.v.copy_(fresh.v)
        q_last.copy_(fresh.q[:, :, -C:])
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, caller_ws_step()), f"replay {i}"
