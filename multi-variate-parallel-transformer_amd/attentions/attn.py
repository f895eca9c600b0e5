"""`flash_mvpa`: the fused MVPA attention operator, served by the gfx950 HIP kernels.

Same call signature, argument meaning and error behaviour as the reference operator
(attentions/attn.py:1317-1366), so `from attentions import flashmvpa` keeps working for
layers/mvpa.py.  Differences in mechanism only: the relative-bias tables [B,H,N,T] and
[B,H,N,C] that the reference materialises in HBM (attentions/attn.py:1305-1314) are never
built - the kernel contracts the query with the small key tables itself.

Forward only: dropout (p_drop > 0), a torch.Generator and autograd are not implemented and
raise NotImplementedError.
"""
from __future__ import annotations

import torch

import mvpa_hip


def flash_mvpa(
    q,            # [B,H,N,Dh]
    q_bias,       # [1,Hkv,1,Dh]  content bias u
    q_btime,      # [1,Hkv,1,Dh]  time bias v
    q_bchan,      # [1,Hkv,1,Dh]  channel bias z
    k_glob,       # [B,Hkv,N,Dh]
    k_time,       # [1,Hkv,T,Dh]
    k_chan,       # [1,Hkv,C,Dh]
    v,            # [B,Hkv,N,Dh]
    causal,
    sm_scale,
    window_size=0,
    p_drop=0.0,
    sequence_parallel=False,
    rel_bias_time=True,
    rel_bias_chan=True,
    generator=None,
    *,
    chan_valid=None,     # extension: [B,C] channel-validity mask (1 = present)
    out=None,            # extension: preallocated output, any [B,H,N,Dh]-indexable view
    kernel=mvpa_hip.KERNEL_AUTO,
):
    if rel_bias_chan or rel_bias_time:
        causal = True                                   # attentions/attn.py:1335-1336
    q_heads, kv_heads = q.shape[1], v.shape[1]
    assert q_heads % kv_heads == 0, "Q heads must be divisible by KV heads."
    n_ctx, time_ctx, chan_ctx = q.shape[2], k_time.shape[2], k_chan.shape[2]
    assert n_ctx == time_ctx * chan_ctx
    assert q.shape[-1] == k_glob.shape[-1] == v.shape[-1]
    assert q.shape[-1] in {16, 32, 64, 128}
    assert time_ctx > 0 and chan_ctx > 0
    if p_drop and p_drop > 0:
        raise NotImplementedError("flash_mvpa: attention dropout is not implemented (forward/eval only)")
    if generator is not None:
        raise NotImplementedError("flash_mvpa: generator is only meaningful with dropout")
    if window_size > 0 and not (rel_bias_chan or rel_bias_time):
        raise NotImplementedError(
            "flash_mvpa: a content window without relative biases (masking instead of zeroing) "
            "is not implemented")
    if torch.is_grad_enabled() and any(
            t.requires_grad for t in (q, q_bias, q_btime, q_bchan, k_glob, k_time, k_chan, v)):
        raise NotImplementedError("flash_mvpa: backward is not implemented; call under torch.no_grad()")
    if not q.is_cuda:
        raise RuntimeError("flash_mvpa needs GPU tensors (there is no CPU path)")
    dh = q.shape[-1]
    return mvpa_hip.mvpa_forward(
        q, k_glob, v,
        q_bias.reshape(kv_heads, dh), q_btime.reshape(kv_heads, dh), q_bchan.reshape(kv_heads, dh),
        k_time.reshape(kv_heads, time_ctx, dh), k_chan.reshape(kv_heads, chan_ctx, dh),
        sm_scale=sm_scale, window=int(window_size), causal=bool(causal), content=True,
        time_bias=bool(rel_bias_time), chan_bias=bool(rel_bias_chan), chan_valid=chan_valid,
        out=out, kernel=kernel)
