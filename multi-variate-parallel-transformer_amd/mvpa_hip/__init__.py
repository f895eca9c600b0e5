"""ctypes binding of libmvpa_hip.so (the C ABI declared in include/mvpa_hip.h).

PyTorch is used only for device memory and streams: every op here hands raw device
pointers and the current HIP stream to the library.  There is no fallback: if the shared
library is missing or an entry point reports an error, the call raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmvpa_hip.so")

MVPA_F32, MVPA_BF16, MVPA_F16 = 0, 1, 2
KERNEL_AUTO, KERNEL_GENERIC, KERNEL_MFMA, KERNEL_MFMA_STEP, KERNEL_MFMA_SPLIT = 0, 1, 2, 3, 4
FLAG_LAST_STEP = 32
FLAG_RING = 64
FLAG_CAUSAL, FLAG_CONTENT, FLAG_TIME_BIAS, FLAG_CHAN_BIAS, FLAG_FP8_QK = 1, 2, 4, 8, 16

ERR_HEAD_DIM, ERR_HEAD_RATIO, ERR_CTX, ERR_SHAPE = -2, -3, -4, -5


class MvpaFwdArgs(ctypes.Structure):
    """Mirror of struct mvpa_fwd_args."""
    _fields_ = [
        ("struct_size", ctypes.c_uint32), ("dtype", ctypes.c_int32),
        ("kernel", ctypes.c_int32), ("flags", ctypes.c_uint32),
        ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("Hkv", ctypes.c_int32),
        ("T", ctypes.c_int32), ("C", ctypes.c_int32), ("Dh", ctypes.c_int32),
        ("window", ctypes.c_int32), ("sm_scale", ctypes.c_float),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("q_stride_b", ctypes.c_int64), ("q_stride_h", ctypes.c_int64), ("q_stride_n", ctypes.c_int64),
        ("k_stride_b", ctypes.c_int64), ("k_stride_h", ctypes.c_int64), ("k_stride_n", ctypes.c_int64),
        ("v_stride_b", ctypes.c_int64), ("v_stride_h", ctypes.c_int64), ("v_stride_n", ctypes.c_int64),
        ("o_stride_b", ctypes.c_int64), ("o_stride_h", ctypes.c_int64), ("o_stride_n", ctypes.c_int64),
        ("bias_u", ctypes.c_void_p), ("bias_v", ctypes.c_void_p), ("bias_z", ctypes.c_void_p),
        ("k_time", ctypes.c_void_p), ("k_chan", ctypes.c_void_p),
        ("chan_valid", ctypes.c_void_p), ("key_bias", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("fp8_q_scale", ctypes.c_void_p), ("fp8_k_scale", ctypes.c_void_p),
        ("split_ws", ctypes.c_void_p), ("n_split", ctypes.c_int32), ("reserved0", ctypes.c_int32),
        ("ring_head", ctypes.c_void_p), ("k_fp8", ctypes.c_void_p),
    ]


class MvpaBwdArgs(ctypes.Structure):
    """Mirror of struct mvpa_bwd_args."""
    _fields_ = (
        [("struct_size", ctypes.c_uint32), ("dtype", ctypes.c_int32), ("flags", ctypes.c_uint32),
         ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("Hkv", ctypes.c_int32),
         ("T", ctypes.c_int32), ("C", ctypes.c_int32), ("Dh", ctypes.c_int32),
         ("window", ctypes.c_int32), ("sm_scale", ctypes.c_float)]
        + [(n, ctypes.c_void_p) for n in ("q", "k", "v", "o", "d_o")]
        + [(f"{t}_stride_{ax}", ctypes.c_int64) for t in ("q", "k", "v", "o", "do") for ax in "bhn"]
        + [(n, ctypes.c_void_p) for n in (
            "bias_u", "bias_v", "bias_z", "k_time", "k_chan", "chan_valid", "key_bias", "lse",
            "dq", "dk", "dv", "dbias_time", "dbias_chan", "ws_delta", "ws_time", "ws_chan", "ws_qu")]
    )


class MvpaError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__(f"libmvpa_hip: {text} (status {status})")
        self.status = status


_lib = None


def load_library() -> ctypes.CDLL:
    """Load the in-tree shared library; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing - build it with `python __graft_entry__.py` "
            "(hipcc --offload-arch=gfx950); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, i64, u32, f32 = (ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64,
                              ctypes.c_uint32, ctypes.c_float)
    lib.mvpa_version.restype = ctypes.c_int
    lib.mvpa_version.argtypes = []
    lib.mvpa_error_string.restype = ctypes.c_char_p
    lib.mvpa_error_string.argtypes = [ctypes.c_int]
    for name in ("mvpa_validate", "mvpa_select_kernel"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.POINTER(MvpaFwdArgs)]
    lib.mvpa_linear_bf16_splitk.restype = ctypes.c_int
    lib.mvpa_linear_bf16_splitk.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, i32, vp, ctypes.c_size_t, vp]
    lib.mvpa_linear_splitk_ws_bytes.restype = ctypes.c_size_t
    lib.mvpa_linear_splitk_ws_bytes.argtypes = [i64, i64, i64, i32]
    lib.mvpa_ring_append_bf16.restype = ctypes.c_int
    lib.mvpa_ring_append_bf16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i64, i64, i64, vp]
    lib.mvpa_split_ws_bytes.restype = ctypes.c_size_t
    lib.mvpa_split_ws_bytes.argtypes = [ctypes.POINTER(MvpaFwdArgs)]
    lib.mvpa_forward.restype = ctypes.c_int
    lib.mvpa_forward.argtypes = [ctypes.POINTER(MvpaFwdArgs), vp]
    lib.mvpa_forward_last_step_static.restype = ctypes.c_int
    lib.mvpa_forward_last_step_static.argtypes = [ctypes.POINTER(MvpaFwdArgs), vp]
    lib.mvpa_static_ws_bytes.restype = ctypes.c_size_t
    lib.mvpa_static_ws_bytes.argtypes = []
    lib.mvpa_static_ws_init.restype = ctypes.c_int
    lib.mvpa_static_ws_init.argtypes = []
    lib.mvpa_backward.restype = ctypes.c_int
    lib.mvpa_backward.argtypes = [ctypes.POINTER(MvpaBwdArgs), vp]
    lib.mvpa_linear_sumsq_parts.restype = ctypes.c_int32
    lib.mvpa_linear_sumsq_parts.argtypes = [i64, i64]
    lib.mvpa_linear_bf16_residual_sumsq.restype = ctypes.c_int
    lib.mvpa_linear_bf16_residual_sumsq.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp]
    lib.mvpa_row_sumsq_bf16.restype = ctypes.c_int
    lib.mvpa_row_sumsq_bf16.argtypes = [vp, vp, i64, i32, i64, vp]
    lib.mvpa_linear_bf16_dual_normed.restype = ctypes.c_int
    lib.mvpa_linear_bf16_dual_normed.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64,
                                                 vp, i32, f32, vp]
    lib.mvpa_linear_f32.restype = ctypes.c_int
    lib.mvpa_linear_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, vp]
    lib.mvpa_fp8_prepare.restype = ctypes.c_int
    lib.mvpa_fp8_prepare.argtypes = [ctypes.POINTER(MvpaFwdArgs), vp, vp, vp, vp]
    lib.mvpa_debug_block_order.restype = ctypes.c_int
    lib.mvpa_debug_block_order.argtypes = [i32, i32, i32, vp, vp]
    lib.mvpa_debug_maps.restype = ctypes.c_int
    lib.mvpa_debug_maps.argtypes = [i32, i32, i32, u32, vp, vp, vp, vp, vp]
    lib.mvpa_linear_bf16.restype = ctypes.c_int
    lib.mvpa_linear_bf16.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, i32, vp]
    lib.mvpa_linear_bf16_dual.restype = ctypes.c_int
    lib.mvpa_linear_bf16_dual.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64, vp]
    lib.mvpa_cosine_rows_bf16.restype = ctypes.c_int
    lib.mvpa_cosine_rows_bf16.argtypes = [vp, vp, vp, i64, i64, i32, i64, i64, i64, i64, ctypes.c_float, vp]
    lib.mvpa_linear_bf16_residual.restype = ctypes.c_int
    lib.mvpa_linear_bf16_residual.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp]
    lib.mvpa_rmsnorm.restype = ctypes.c_int
    lib.mvpa_rmsnorm.argtypes = [vp, vp, vp, i64, i32, i64, i64, f32, i32, i32, vp]
    lib.mvpa_add3_bf16.restype = ctypes.c_int
    lib.mvpa_add3_bf16.argtypes = [vp, vp, vp, vp, i64, vp]
    lib.mvpa_add3_rmsnorm_bf16.restype = ctypes.c_int
    lib.mvpa_add3_rmsnorm_bf16.argtypes = [vp, vp, vp, vp, vp, vp, i64, i32, f32, vp]
    lib.mvpa_wavedec_db4.restype = ctypes.c_int
    lib.mvpa_wavedec_db4.argtypes = [vp, vp, i64, i32, i32, i32, i64, vp]
    if lib.mvpa_version() != 3:
        raise RuntimeError("libmvpa_hip ABI version mismatch")
    _lib = lib
    return lib


def error_string(status: int) -> str:
    return load_library().mvpa_error_string(status).decode()


def _check(status: int) -> None:
    """Map library status codes onto the reference's exception types
    (AssertionError for the shape asserts of attentions/attn.py:1041-1045, 1339, 1344)."""
    if status == 0:
        return
    text = error_string(status)
    if status in (ERR_HEAD_DIM, ERR_HEAD_RATIO, ERR_CTX, ERR_SHAPE):
        raise AssertionError(f"libmvpa_hip: {text} (status {status})")
    raise MvpaError(status, text)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of torch's current stream on the current device (the raw getter skips building a
    Stream object: this runs once per launch)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return MVPA_F32
    if dt == torch.bfloat16:
        return MVPA_BF16
    if dt == torch.float16:
        return MVPA_F16
    raise TypeError(f"libmvpa_hip supports float32, bfloat16 and float16, got {dt}")


def _need_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("libmvpa_hip ops need tensors in GPU memory (there is no CPU path)")


def make_args(q, k, v, out, u, vb, z, k_time, k_chan, *, T: int, C: int,
              sm_scale: float, window: int = 10, flags: int = 15,
              chan_valid=None, key_bias=None, lse=None, kernel: int = KERNEL_AUTO,
              fp8_q_scale=None, fp8_k_scale=None, split_ws=None, n_split: int = 0,
              ring_head=None, k_fp8=None) -> MvpaFwdArgs:
    """Fill the argument block from [B,H,N,Dh]-indexable tensors (any strides with a unit
    last stride).  Accepts meta/CPU tensors too so validation can be exercised without a GPU."""
    a = MvpaFwdArgs()
    a.struct_size = ctypes.sizeof(MvpaFwdArgs)
    a.dtype = _dtype_code(q.dtype)
    a.kernel = kernel
    a.flags = flags
    a.B, a.H, _, a.Dh = q.shape
    a.Hkv = k.shape[1]
    a.T, a.C = T, C
    a.window = window
    a.sm_scale = sm_scale
    for name, t in (("q", q), ("k", k), ("v", v), ("o", out)):
        if t.stride(-1) != 1:
            raise ValueError(f"{name}: last dim must be contiguous")
        setattr(a, name, t.data_ptr())
        setattr(a, f"{name}_stride_b", t.stride(0))
        setattr(a, f"{name}_stride_h", t.stride(1))
        setattr(a, f"{name}_stride_n", t.stride(2))
    a.bias_u, a.bias_v, a.bias_z = u.data_ptr(), vb.data_ptr(), z.data_ptr()
    a.k_time, a.k_chan = k_time.data_ptr(), k_chan.data_ptr()
    a.chan_valid = chan_valid.data_ptr() if chan_valid is not None else None
    a.key_bias = key_bias.data_ptr() if key_bias is not None else None
    a.lse = lse.data_ptr() if lse is not None else None
    a.fp8_q_scale = fp8_q_scale.data_ptr() if fp8_q_scale is not None else None
    a.fp8_k_scale = fp8_k_scale.data_ptr() if fp8_k_scale is not None else None
    a.split_ws = split_ws.data_ptr() if split_ws is not None else None
    a.n_split = n_split
    a.ring_head = ring_head.data_ptr() if ring_head is not None else None
    a.k_fp8 = k_fp8.data_ptr() if k_fp8 is not None else None
    return a


def default_key_splits(B: int, H: int, T: int) -> int:
    """Runs of key steps a last-step launch is cut into: about one workgroup per CU (256), at
    least 8 key steps per run, no empty run.  Measured: B1 H16 C128 T512 Dh128 2.50 ms unsplit,
    0.11 ms at 16 runs, 0.14 at 32; B4 H16 C64 T128 0.071 ms unsplit, 0.034 at 4 runs, 0.050 at 16."""
    n = max(1, min(T // 8, 256 // max(1, B * H)))
    while n > 1 and (n - 1) * ((T + n - 1) // n) >= T:
        n -= 1
    return n


def mvpa_forward(q, k, v, u, vb, z, k_time, k_chan, *, sm_scale: Optional[float] = None,
                 window: int = 10, causal: bool = True, content: bool = True,
                 time_bias: bool = True, chan_bias: bool = True,
                 chan_valid: Optional[torch.Tensor] = None,
                 key_bias: Optional[torch.Tensor] = None, return_lse: bool = False,
                 kernel: int = KERNEL_AUTO, out: Optional[torch.Tensor] = None,
                 fp8_qk: bool = False, last_step_only: bool = False,
                 key_splits: Optional[int] = None, ring_head: Optional[torch.Tensor] = None,
                 static_ws: bool = False):
    """Fused MVPA forward on the GPU.

    q [B,H,N,Dh]; k, v [B,Hkv,N,Dh]; u, vb, z [Hkv,Dh]; k_time [Hkv,T,Dh]; k_chan [Hkv,C,Dh];
    chan_valid [B,C] bool/uint8; key_bias [B,N] float32 additive.  Returns out [B,H,N,Dh] in
    q's dtype (and the base-2 log-sum-exp [B,H,N] float32 if asked).

    last_step_only: q holds only the C queries of the last time step ([B,H,C,Dh]) while k, v hold
    all T*C rows (cached steps followed by the new one); out is [B,H,C,Dh].  One step of
    incremental decoding.  key_splits: the number of runs the T key steps are cut into, each run
    on workgroups of its own, merged by a second kernel (bf16 MFMA kernel only; None picks
    default_key_splits, 1 keeps one workgroup per (b, h) on the whole cache).
    ring_head (with last_step_only, bf16): a one-element int32 device tensor; the T time steps of
    k and v are then the slots of a ring, slot ring_head holding the newest step and slot s the one
    (ring_head - s) mod T steps older.  The kernel reads it from device memory, so a captured
    graph of the call follows a cache that moves on.
    static_ws (with last_step_only and more than one key run): the runs' partial results go through
    the workspace built into the library (mvpa_forward_last_step_static) instead of one allocated
    here; with `out` given the call then allocates no device memory at all.
    """
    lib = load_library()
    _need_cuda(q, k, v, u, vb, z, k_time, k_chan, chan_valid, key_bias)
    B, H, Nq, Dh = q.shape
    assert k.shape[-1] == Dh and v.shape[-1] == Dh, "head dims of q, k, v differ"
    T, C = k_time.shape[-2], k_chan.shape[-2]
    N = T * C
    assert k.shape[2] == N and v.shape[2] == N, "k and v must hold T*C rows"
    assert Nq == (C if last_step_only else N), "q must hold T*C rows (C with last_step_only)"
    if last_step_only and not causal:
        raise ValueError("last_step_only needs the time-causal mask")
    dt = q.dtype
    u, vb, z = (t.to(dt).contiguous() for t in (u, vb, z))
    k_time, k_chan = k_time.to(dt).contiguous(), k_chan.to(dt).contiguous()
    if out is None:
        out = torch.empty((B, H, Nq, Dh), dtype=dt, device=q.device)
    if chan_valid is not None:
        chan_valid = chan_valid.to(torch.uint8).contiguous()
        assert chan_valid.shape == (B, C)
    if key_bias is not None:
        key_bias = key_bias.to(torch.float32).contiguous()
        assert key_bias.shape == (B, N)
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device=q.device) if return_lse else None
    flags = ((FLAG_CAUSAL if causal else 0) | (FLAG_CONTENT if content else 0) |
             (FLAG_TIME_BIAS if time_bias else 0) | (FLAG_CHAN_BIAS if chan_bias else 0) |
             (FLAG_FP8_QK if fp8_qk else 0) | (FLAG_LAST_STEP if last_step_only else 0) |
             (FLAG_RING if ring_head is not None else 0))
    if ring_head is not None:
        if not last_step_only:
            raise ValueError("ring_head needs last_step_only")
        if ring_head.dtype != torch.int32 or not ring_head.is_cuda or ring_head.numel() != 1:
            raise TypeError("ring_head: one int32 element on the GPU")
    s = (1.0 / Dh ** 0.5) if sm_scale is None else float(sm_scale)
    q_scale = k_scale = k8 = None
    if fp8_qk:
        # per-head amax scales and the e4m3 copy of the keys, by the library (mvpa_fp8_prepare):
        # the kernel rounds (q+u)*s*log2(e)/q_scale to e4m3 itself and multiplies it with k/k_scale
        q_scale = torch.empty(H, dtype=torch.float32, device=q.device)
        k_scale = torch.empty(k.shape[1], dtype=torch.float32, device=q.device)
        if not last_step_only and 32 < C <= 128 and Dh in (64, 128):      # shapes of the column-split build
            k8 = torch.empty((B, k.shape[1], N, Dh), dtype=torch.uint8, device=q.device)
        pa = make_args(q, k, v, out, u, vb, z, k_time, k_chan, T=T, C=C, sm_scale=s, window=window,
                       flags=flags)
        _check(lib.mvpa_fp8_prepare(ctypes.byref(pa), q_scale.data_ptr(), k_scale.data_ptr(),
                                    k8.data_ptr() if k8 is not None else None, _stream()))
    a = make_args(q, k, v, out, u, vb, z, k_time, k_chan, T=T, C=C, sm_scale=s, window=window,
                  flags=flags, chan_valid=chan_valid, key_bias=key_bias, lse=lse, kernel=kernel,
                  fp8_q_scale=q_scale, fp8_k_scale=k_scale, ring_head=ring_head, k_fp8=k8)
    if last_step_only and lib.mvpa_select_kernel(ctypes.byref(a)) == KERNEL_MFMA:
        n = default_key_splits(B, H, T) if key_splits is None else int(key_splits)
        if n > 1:
            a.n_split = n
            if static_ws:
                static_ws_init(q.device)
                _check(lib.mvpa_forward_last_step_static(ctypes.byref(a), _stream()))
                return (out, lse) if return_lse else out
            ws = torch.empty(lib.mvpa_split_ws_bytes(ctypes.byref(a)), dtype=torch.uint8, device=q.device)
            a.split_ws = ws.data_ptr()
    if static_ws:
        raise ValueError("static_ws needs last_step_only on the bf16 matrix-core kernel with more than one key run")
    _check(lib.mvpa_forward(ctypes.byref(a), _stream()))
    return (out, lse) if return_lse else out


_static_ws_ready = set()


def static_ws_init(device=None) -> None:
    """Set-up of mvpa_forward_last_step_static on a GPU (mvpa_static_ws_init with that GPU
    current): call it once per GPU before recording the step into a graph."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    if idx in _static_ws_ready:
        return
    with torch.cuda.device(idx):
        _check(load_library().mvpa_static_ws_init())
    _static_ws_ready.add(idx)


def mvpa_backward(q, k, v, o, d_o, lse, u, vb, z, k_time, k_chan, *,
                  sm_scale: Optional[float] = None, window: int = 10, causal: bool = True,
                  content: bool = True, time_bias: bool = True, chan_bias: bool = True,
                  chan_valid: Optional[torch.Tensor] = None,
                  key_bias: Optional[torch.Tensor] = None):
    """Backward of mvpa_forward at the boundary of the reference's FlashMVPA.backward
    (attentions/attn.py:1140-1302).  Shapes as in mvpa_forward; o, lse are the forward's results.
    Returns fp32 tensors (dq_content [B,H,N,Dh], dk [B,Hkv,N,Dh], dv [B,Hkv,N,Dh],
    dbias_time [B,H,N,T], dbias_chan [B,H,N,C])."""
    lib = load_library()
    _need_cuda(q, k, v, o, d_o, lse, u, vb, z, k_time, k_chan, chan_valid, key_bias)
    B, H, N, Dh = q.shape
    Hkv = k.shape[1]
    T, C = k_time.shape[-2], k_chan.shape[-2]
    assert N == T * C, "N must equal T*C"
    dt = q.dtype
    u, vb, z = (t.to(dt).contiguous() for t in (u, vb, z))
    k_time, k_chan = k_time.to(dt).contiguous(), k_chan.to(dt).contiguous()
    o, d_o = o.to(dt), d_o.to(dt)
    lse = lse.to(torch.float32).contiguous()
    if chan_valid is not None:
        chan_valid = chan_valid.to(torch.uint8).contiguous()
    if key_bias is not None:
        key_bias = key_bias.to(torch.float32).contiguous()
    f32 = dict(dtype=torch.float32, device=q.device)
    dq = torch.empty((B, H, N, Dh), **f32)
    dk = torch.empty((B, Hkv, N, Dh), **f32)
    dv = torch.empty((B, Hkv, N, Dh), **f32)
    dbt = torch.empty((B, H, N, T), **f32)
    dbc = torch.empty((B, H, N, C), **f32)
    ws_delta = torch.empty((B, H, N), **f32)
    ws_time = torch.empty((B, H, N, T), **f32)
    ws_chan = torch.empty((B, H, N, (C + 3) // 4 * 4), **f32)
    ws_qu = torch.empty((B, H, N, Dh), dtype=dt, device=q.device)
    a = MvpaBwdArgs()
    a.struct_size = ctypes.sizeof(MvpaBwdArgs)
    a.dtype = _dtype_code(dt)
    a.flags = ((FLAG_CAUSAL if causal else 0) | (FLAG_CONTENT if content else 0) |
               (FLAG_TIME_BIAS if time_bias else 0) | (FLAG_CHAN_BIAS if chan_bias else 0))
    a.B, a.H, a.Hkv, a.T, a.C, a.Dh = B, H, Hkv, T, C, Dh
    a.window = window
    a.sm_scale = (1.0 / Dh ** 0.5) if sm_scale is None else float(sm_scale)
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o), ("do", d_o)):
        if t.stride(-1) != 1:
            raise ValueError(f"{name}: last dim must be contiguous")
        setattr(a, "d_o" if name == "do" else name, t.data_ptr())
        for ax, st in zip("bhn", t.stride()[:3]):
            setattr(a, f"{name}_stride_{ax}", st)
    a.bias_u, a.bias_v, a.bias_z = u.data_ptr(), vb.data_ptr(), z.data_ptr()
    a.k_time, a.k_chan = k_time.data_ptr(), k_chan.data_ptr()
    a.chan_valid = chan_valid.data_ptr() if chan_valid is not None else None
    a.key_bias = key_bias.data_ptr() if key_bias is not None else None
    a.lse = lse.data_ptr()
    a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    a.dbias_time, a.dbias_chan = dbt.data_ptr(), dbc.data_ptr()
    a.ws_delta, a.ws_time, a.ws_chan = ws_delta.data_ptr(), ws_time.data_ptr(), ws_chan.data_ptr()
    a.ws_qu = ws_qu.data_ptr()
    _check(lib.mvpa_backward(ctypes.byref(a), _stream()))
    return dq, dk, dv, dbt, dbc


def debug_maps(T: int, C: int, window: int = 10, flags: int = 15, chan_valid=None,
               device="cuda"):
    """Index and mask maps as the kernels compute them: (time_idx, chan_idx, mask_bits),
    each [N,N]."""
    lib = load_library()
    N = T * C
    ti = torch.empty((N, N), dtype=torch.int32, device=device)
    ci = torch.empty((N, N), dtype=torch.int32, device=device)
    mb = torch.empty((N, N), dtype=torch.uint8, device=device)
    cv = chan_valid.to(torch.uint8).contiguous() if chan_valid is not None else None
    _check(lib.mvpa_debug_maps(T, C, window, flags, cv.data_ptr() if cv is not None else None,
                               ti.data_ptr(), ci.data_ptr(), mb.data_ptr(), _stream()))
    return ti, ci, mb


def linear_residual_supported(M: int, K: int) -> bool:
    """Shapes mvpa_linear_bf16_residual takes (the large-tile kernel: see include/mvpa_hip.h)."""
    return M >= 512 and K % 32 == 0 and K >= 96


def linear_dual_supported(M: int, K: int) -> bool:
    """Shapes mvpa_linear_bf16_dual takes (see include/mvpa_hip.h)."""
    return M >= 512 and K % 64 == 0 and K >= 128


def linear_dual(x: torch.Tensor, w_plain: torch.Tensor, w_gated: torch.Tensor,
                out_plain: Optional[torch.Tensor] = None, out_gated: Optional[torch.Tensor] = None,
                sumsq: Optional[torch.Tensor] = None, eps: float = 1e-5):
    """(x @ w_plain.T, silu(x @ gate.T) * (x @ up.T)) from ONE launch; w_gated stacks [gate; up]
    rows.  x is [rows, K] (or any shape with K last, contiguous); the outputs are 2-D, and either
    may be a given [rows, N] view with unit last stride (a column slice of a wider buffer).
    sumsq ([rows, parts] fp32, from row_sumsq or linear(..., sumsq_out=True)): x holds RAW rows
    whose RMSNorm is applied in the epilogue - every output row is scaled by
    rsqrt(sum(sumsq[row]) / K + eps); the weights must carry the norm's weight in their columns."""
    lib = load_library()
    _need_cuda(x, w_plain, w_gated)
    if x.dtype != torch.bfloat16 or w_plain.dtype != torch.bfloat16 or w_gated.dtype != torch.bfloat16:
        raise TypeError("linear_dual: bf16 only")
    K = x.shape[-1]
    x2 = x if x.dim() == 2 and x.stride(-1) == 1 else x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    M, N0, N1 = x2.shape[0], w_plain.shape[0], w_gated.shape[0] // 2
    assert w_plain.shape[1] == K and w_gated.shape[1] == K and w_plain.stride(1) == 1 and w_gated.stride(1) == 1
    outs = []
    for o, n in ((out_plain, N0), (out_gated, N1)):
        if o is None:
            o = torch.empty((M, n), dtype=torch.bfloat16, device=x.device)
        elif o.dim() != 2 or tuple(o.shape) != (M, n) or o.stride(1) != 1 or o.dtype != torch.bfloat16:
            raise ValueError("linear_dual: outputs must be bf16 [rows, N] tensors or views with unit last stride")
        outs.append(o)
    if sumsq is not None:
        if sumsq.dtype != torch.float32 or sumsq.dim() != 2 or sumsq.shape[0] != M or not sumsq.is_contiguous():
            raise ValueError("linear_dual: sumsq must be a contiguous fp32 [rows, parts] tensor")
        _need_cuda(sumsq)
        _check(lib.mvpa_linear_bf16_dual_normed(
            x2.data_ptr(), w_plain.data_ptr(), outs[0].data_ptr(), w_gated.data_ptr(), outs[1].data_ptr(),
            M, N0, N1, K, x2.stride(0), w_plain.stride(0), outs[0].stride(0), w_gated.stride(0),
            outs[1].stride(0), sumsq.data_ptr(), sumsq.shape[1], float(eps), _stream()))
        return outs[0], outs[1]
    _check(lib.mvpa_linear_bf16_dual(x2.data_ptr(), w_plain.data_ptr(), outs[0].data_ptr(), w_gated.data_ptr(),
                                     outs[1].data_ptr(), M, N0, N1, K, x2.stride(0), w_plain.stride(0),
                                     outs[0].stride(0), w_gated.stride(0), outs[1].stride(0), _stream()))
    return outs[0], outs[1]


def row_sumsq(x: torch.Tensor) -> torch.Tensor:
    """[rows, 1] fp32 sums of squares of bf16 rows ([rows, cols] view, unit last stride, cols a
    multiple of 8): the row statistics an RMSNorm needs, in the form linear_dual(sumsq=...) takes."""
    lib = load_library()
    _need_cuda(x)
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.stride(1) != 1:
        raise TypeError("row_sumsq: a bf16 [rows, cols] tensor or view with unit last stride")
    out = torch.empty((x.shape[0], 1), dtype=torch.float32, device=x.device)
    _check(lib.mvpa_row_sumsq_bf16(x.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], x.stride(0), _stream()))
    return out


def linear_norm_fused_supported(M: int, K: int, N: int) -> bool:
    """Shapes for which the tail product can write row statistics (linear(..., sumsq_out=True))
    and the dual product can consume them (linear_dual(sumsq=...))."""
    return M >= 512 and K % 64 == 0 and K >= 128 and N % 8 == 0


def linear(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None,
           gated: bool = False, split_k: Optional[bool] = None,
           residual: Optional[torch.Tensor] = None, sumsq_out: bool = False) -> torch.Tensor:
    """y = x @ weight.T in bf16 on MFMA.  gated=True: weight stacks [gate; up] rows and the
    result is silu(x@gate.T) * (x@up.T).  split_k: the K-split kernel pair through a workspace
    (at most 128 rows); None picks it for K >= 1536 and at most 4096 rows of weight.
    x may be a 2-D row-pitched view (unit last stride), out a 2-D view [rows, N] likewise.
    residual: [rows, N] bf16 added in the product's epilogue (shapes for which
    linear_residual_supported holds; otherwise MvpaError).
    sumsq_out (with residual): also returns the partial sums of squares of the output rows,
    [rows, parts] fp32 - (out, sumsq) comes back - for a later linear_dual(sumsq=...)."""
    lib = load_library()
    _need_cuda(x, weight)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("linear: bf16 only")
    K = x.shape[-1]
    x2 = x if x.dim() == 2 and x.stride(-1) == 1 else x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    assert weight.shape[1] == K and weight.stride(1) == 1
    M = x2.shape[0]
    N = weight.shape[0] // 2 if gated else weight.shape[0]
    given = out is not None
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    else:
        if out.dim() != 2 or tuple(out.shape) != (M, N) or out.stride(1) != 1 or out.dtype != torch.bfloat16:
            raise ValueError("linear: out must be a bf16 [rows, N] tensor or view with unit last stride")
    if residual is not None:
        if gated or split_k:
            raise ValueError("linear: residual goes with the plain product only")
        r2 = residual.reshape(M, N) if residual.dim() != 2 else residual
        if tuple(r2.shape) != (M, N) or r2.stride(1) != 1 or r2.dtype != torch.bfloat16:
            raise ValueError("linear: residual must be bf16 [rows, N] with unit last stride")
        _need_cuda(r2)
        if sumsq_out:
            ss = torch.empty((M, lib.mvpa_linear_sumsq_parts(M, N)), dtype=torch.float32, device=x.device)
            _check(lib.mvpa_linear_bf16_residual_sumsq(x2.data_ptr(), weight.data_ptr(), r2.data_ptr(), out.data_ptr(),
                                                       ss.data_ptr(), M, N, K, x2.stride(0), weight.stride(0),
                                                       r2.stride(0), out.stride(0), _stream()))
            return (out if given else out.view(*x.shape[:-1], N)), ss
        _check(lib.mvpa_linear_bf16_residual(x2.data_ptr(), weight.data_ptr(), r2.data_ptr(), out.data_ptr(),
                                             M, N, K, x2.stride(0), weight.stride(0), r2.stride(0),
                                             out.stride(0), _stream()))
        return out if given else out.view(*x.shape[:-1], N)
    if sumsq_out:
        raise ValueError("linear: sumsq_out goes with residual")
    if split_k is None:
        # measured on graph replays (GPU time): [128x2048]x[2048x4096] 22.9 -> 18.6 us,
        # [128x5632]x[5632x2048] 58.1 -> 21.0 us, [64x1728]x[1728x768] 13.2 -> 10.0 us; the wide
        # gate/up product ([128x2048]x[2048x11264]) is better off in one kernel (33.7 against 41.6 us)
        split_k = M <= 128 and K >= 1536 and weight.shape[0] <= 4096
    if split_k:
        ws = torch.empty(lib.mvpa_linear_splitk_ws_bytes(M, N, K, 1 if gated else 0), dtype=torch.uint8,
                         device=x.device)
        _check(lib.mvpa_linear_bf16_splitk(x2.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K,
                                           x2.stride(0), weight.stride(0), out.stride(0),
                                           1 if gated else 0, ws.data_ptr(), ws.numel(), _stream()))
        return out if given else out.view(*x.shape[:-1], N)
    _check(lib.mvpa_linear_bf16(x2.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K,
                                x2.stride(0), weight.stride(0), out.stride(0),
                                1 if gated else 0, _stream()))
    return out if given else out.view(*x.shape[:-1], N)


def linear_f32(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x @ weight.T in fp32 on the GPU library (x: any leading shape, K last)."""
    lib = load_library()
    _need_cuda(x, weight)
    if x.dtype != torch.float32 or weight.dtype != torch.float32:
        raise TypeError("linear_f32: fp32 only")
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    w = weight if weight.stride(-1) == 1 else weight.contiguous()
    assert w.shape[1] == K
    M, N = x2.shape[0], w.shape[0]
    out = torch.empty((M, N), dtype=torch.float32, device=x.device)
    _check(lib.mvpa_linear_f32(x2.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, x2.stride(0),
                               w.stride(0), out.stride(0), _stream()))
    return out.view(*x.shape[:-1], N)


def cosine_similarity_steps(nxt: torch.Tensor, pred: torch.Tensor, eps: float = 1e-8) -> torch.Tensor:
    """torch.cosine_similarity(nxt[:, 1:], pred[:, :-1], dim=-1) for two bf16 tensors [B, T, C, E]
    (the reference's generative score, models/mvpformer.py:749-764) in one kernel, fp32 result
    [B, T-1, C]."""
    lib = load_library()
    _need_cuda(nxt, pred)
    if nxt.dtype != torch.bfloat16 or pred.dtype != torch.bfloat16:
        raise TypeError("cosine_similarity_steps: bf16 only")
    if nxt.shape != pred.shape or nxt.dim() != 4:
        raise ValueError("cosine_similarity_steps: two tensors [B, T, C, E] of one shape")
    nxt, pred = nxt.contiguous(), pred.contiguous()
    B, T, C, E = nxt.shape
    out = torch.empty((B, max(T - 1, 0), C), dtype=torch.float32, device=nxt.device)
    if T > 1 and B > 0 and C > 0:
        a = nxt[:, 1:]
        _check(lib.mvpa_cosine_rows_bf16(a.data_ptr(), pred.data_ptr(), out.data_ptr(), B, (T - 1) * C, E,
                                         E, E, T * C * E, T * C * E, eps, _stream()))
    return out


def _as_f32_weight(weight: torch.Tensor) -> torch.Tensor:
    """fp32 contiguous copy of a (norm) weight, kept on the tensor object and refreshed when the
    tensor is modified in place, so a bf16 module does not convert its weight on every call."""
    if weight.dtype == torch.float32 and weight.is_contiguous():
        return weight.detach()
    cached = getattr(weight, "_mvpa_f32", None)
    if cached is not None and cached[0] == weight._version and cached[1].device == weight.device:
        return cached[1]
    w32 = weight.detach().to(torch.float32).contiguous()
    try:
        weight._mvpa_f32 = (weight._version, w32)
    except AttributeError:
        pass
    return w32


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5,
            out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last dim.  x may be a 2-D row-pitched view (unit last stride); `out`, if
    given, is a 2-D tensor/view [rows, cols] with unit last stride."""
    lib = load_library()
    _need_cuda(x, weight)
    cols = x.shape[-1]
    if x.dim() == 2 and x.stride(-1) == 1:
        x2 = x
    else:
        x2 = x.contiguous().view(-1, cols)
    rows = x2.shape[0]
    od = out_dtype or (out.dtype if out is not None else x.dtype)
    if out is None:
        y = torch.empty(x.shape, dtype=od, device=x.device)
        y2 = y.view(-1, cols)
    else:
        y = y2 = out
        assert out.dim() == 2 and out.shape == (rows, cols) and out.stride(-1) == 1
    w = _as_f32_weight(weight)
    _check(lib.mvpa_rmsnorm(x2.data_ptr(), w.data_ptr(), y2.data_ptr(), rows, cols,
                            x2.stride(0), y2.stride(0), eps, _dtype_code(x.dtype), _dtype_code(od),
                            _stream()))
    return y


def ring_append(k_new: torch.Tensor, v_new: torch.Tensor, k_ring: torch.Tensor, v_ring: torch.Tensor,
                head32: torch.Tensor) -> None:
    """Write one time step ([B,Hkv,C,Dh] views of equal strides, bf16) into slot head32[0] of the
    contiguous ring buffers [B,Hkv,steps,C,Dh]; the slot is read on the device."""
    lib = load_library()
    _need_cuda(k_new, v_new, k_ring, v_ring, head32)
    B, Hkv, C, Dh = k_new.shape
    assert v_new.shape == k_new.shape and k_new.stride() == v_new.stride() and k_new.stride(3) == 1
    assert k_ring.is_contiguous() and v_ring.is_contiguous() and k_ring.shape == v_ring.shape
    assert k_ring.shape[0] == B and k_ring.shape[1] == Hkv and tuple(k_ring.shape[3:]) == (C, Dh)
    assert k_new.dtype == v_new.dtype == k_ring.dtype == v_ring.dtype == torch.bfloat16
    assert head32.dtype == torch.int32
    _check(lib.mvpa_ring_append_bf16(k_new.data_ptr(), v_new.data_ptr(), k_ring.data_ptr(), v_ring.data_ptr(),
                                     head32.data_ptr(), B, Hkv, C, Dh, k_ring.shape[2],
                                     k_new.stride(0), k_new.stride(1), k_new.stride(2), _stream()))


def add3(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    lib = load_library()
    _need_cuda(a, b, c)
    a, b, c = a.contiguous(), b.contiguous(), c.contiguous()
    assert a.dtype == b.dtype == c.dtype == torch.bfloat16 and a.shape == b.shape == c.shape
    out = torch.empty_like(a)
    _check(lib.mvpa_add3_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), out.data_ptr(),
                              a.numel(), _stream()))
    return out


def add3_rmsnorm(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, weight: torch.Tensor,
                 eps: float):
    """(a + b + c, RMSNorm(a + b + c) * weight) in one pass; bit-identical to add3 followed by
    rmsnorm.  Falls back to the two separate kernels when the row length is not a multiple of 8."""
    lib = load_library()
    _need_cuda(a, b, c, weight)
    a, b, c = a.contiguous(), b.contiguous(), c.contiguous()
    assert a.dtype == b.dtype == c.dtype == torch.bfloat16 and a.shape == b.shape == c.shape
    cols = a.shape[-1]
    if cols % 8 != 0:
        total = add3(a, b, c)
        return total, rmsnorm(total, weight, eps)
    w = _as_f32_weight(weight)
    total, normed = torch.empty_like(a), torch.empty_like(a)
    _check(lib.mvpa_add3_rmsnorm_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), w.data_ptr(),
                                      total.data_ptr(), normed.data_ptr(), a.numel() // cols, cols,
                                      float(eps), _stream()))
    return total, normed


def dwt_sizes(size_input: int):
    """Coefficient sizes per level for db4 / periodic extension and the maximum useful depth
    floor(log2(L/7)) (models/fftencoder.py:70-78)."""
    import math
    levels = max(0, int(math.floor(math.log2(size_input / 7))))
    sizes, n = [], size_input
    for _ in range(levels):
        n = (n + 7) // 2
        sizes.append(n)
    sizes.append(n)
    return levels, sizes


def wavedec_db4(x: torch.Tensor, pitch: Optional[int] = None, zero_pad: bool = True) -> torch.Tensor:
    """x [M,L] float32 -> coefficients [M,dwt_size] float32, ordered [cA_L, cD_L, .., cD_1].
    With `pitch` the result is a [M,dwt_size] view of a [M,pitch] buffer, zero-filled unless
    zero_pad is False (the columns past dwt_size are then undefined)."""
    lib = load_library()
    _need_cuda(x)
    x = x.to(torch.float32).contiguous()
    M, L = x.shape
    levels, sizes = dwt_sizes(L)
    total = sum(sizes)
    ldc = total if pitch is None else pitch
    buf = (torch.empty if ldc == total or not zero_pad else torch.zeros)((M, ldc), dtype=torch.float32, device=x.device)
    _check(lib.mvpa_wavedec_db4(x.data_ptr(), buf.data_ptr(), M, L, levels, total, ldc, _stream()))
    return buf[:, :total]
