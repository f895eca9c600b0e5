"""`flash_mvpa`: the fused MVPA attention operator, served by the gfx950 HIP kernels.

Same call signature, argument meaning and error behaviour as the reference operator
(attentions/attn.py:1317-1366), so `from attentions import flashmvpa` keeps working for
layers/mvpa.py.  Differences in mechanism only: the relative-bias tables [B,H,N,T] and
[B,H,N,C] that the reference materialises in HBM (attentions/attn.py:1305-1314) are never
built - the kernel contracts the query with the small key tables itself.

Autograd: when an input requires grad the call goes through `FlashMVPA`, whose backward runs
`mvpa_backward` (the boundary of the reference's FlashMVPA.backward, attentions/attn.py:1140-1302)
and finishes the bias-table gradients with the matrix products that autograd applies to
attentions/attn.py:1305-1314.  Attention dropout (p_drop > 0, optionally with a torch.Generator)
drops whole key time steps and channels as the reference's kernel does; since the soft-max sum
ignores the masks it is applied to the values in front of the kernel (dropout_key_scale).
"""
from __future__ import annotations

import torch

import mvpa_hip


class FlashMVPA(torch.autograd.Function):
    """Differentiable fused MVPA.  forward saves o and the base-2 log-sum-exp (the reference
    saves o and L, attentions/attn.py:1124-1137); nothing of size N x N is kept."""

    @staticmethod
    def forward(ctx, q, u, vb, z, k, k_time, k_chan, v, causal, sm_scale, window, time_bias,
                chan_bias, chan_valid, content=True, key_bias=None):
        out, lse = mvpa_hip.mvpa_forward(q, k, v, u, vb, z, k_time, k_chan, sm_scale=sm_scale,
                                         window=window, causal=causal, content=content,
                                         time_bias=time_bias, chan_bias=chan_bias,
                                         chan_valid=chan_valid, key_bias=key_bias, return_lse=True)
        ctx.save_for_backward(q, u, vb, z, k, k_time, k_chan, v, out, lse)
        ctx.conf = (causal, sm_scale, window, time_bias, chan_bias, chan_valid, content, key_bias)
        return out

    @staticmethod
    def backward(ctx, d_out):
        q, u, vb, z, k, k_time, k_chan, v, out, lse = ctx.saved_tensors
        causal, sm_scale, window, time_bias, chan_bias, chan_valid, content, key_bias = ctx.conf
        dq_c, dk, dv, dbt, dbc = mvpa_hip.mvpa_backward(
            q, k, v, out, d_out.contiguous(), lse, u, vb, z, k_time, k_chan, sm_scale=sm_scale,
            window=window, causal=causal, content=content, time_bias=time_bias, chan_bias=chan_bias,
            chan_valid=chan_valid, key_bias=key_bias)
        B, H, N, Dh = q.shape
        Hkv = k.shape[1]
        grp = H // Hkv
        rows = grp * N                                  # the query rows of a kv head, heads side by side
        dq = dq_c.view(B, Hkv, rows, Dh)
        du = dq.sum(dim=(0, 2)) if content else torch.zeros_like(u, dtype=torch.float32)
        # bf16 runs take these products in bf16 (fp32 accumulation), as the kernels take theirs
        cd = torch.bfloat16 if q.dtype == torch.bfloat16 else torch.float32
        q2 = q.reshape(B, Hkv, rows, Dh)

        # Per kv head g the table is (q + bias) @ table[g]^T, so with its gradient G [rows, J]:
        #   d(q + bias) = G @ table[g]            - one batched product over (b, g), and
        #   d table[g]  = sum_b G^T @ (q + bias)  - one batched product with G read transposed in
        # place, then a sum over b (an einsum over (b, r, n) would first copy G, the largest tensor
        # of the backward, into a [g, (b r n), J] layout).  A bias term that is switched off takes
        # no part in the forward: its table, its query bias and the query get nothing through it.
        def finish(grad_table, table, bias):
            g2 = grad_table.view(B, Hkv, rows, -1).to(cd)
            dq_share = torch.matmul(g2, table.to(cd)).float()          # [B,Hkv,rows,Dh]
            qb = (q2.float() + bias.float()[None, :, None, :]).to(cd)
            dtab = torch.matmul(g2.transpose(2, 3), qb).float().sum(0)  # [Hkv,J,Dh]
            return dq_share, dq_share.sum(dim=(0, 2)), dtab

        if time_bias:
            dq_t, dvb, dk_time = finish(dbt, k_time, vb)
            dq = dq + dq_t
        else:
            dvb, dk_time = torch.zeros_like(vb, dtype=torch.float32), torch.zeros_like(k_time, dtype=torch.float32)
        if chan_bias:
            dq_ch, dz, dk_chan = finish(dbc, k_chan, z)
            dq = dq + dq_ch
        else:
            dz, dk_chan = torch.zeros_like(z, dtype=torch.float32), torch.zeros_like(k_chan, dtype=torch.float32)
        return (dq.view(B, H, N, Dh).to(q.dtype), du.to(u.dtype), dvb.to(vb.dtype), dz.to(z.dtype),
                dk.to(k.dtype), dk_time.to(k_time.dtype), dk_chan.to(k_chan.dtype), dv.to(v.dtype),
                None, None, None, None, None, None, None, None)


def dropout_key_scale(p_drop, time_ctx, chan_ctx, device, generator=None, time_keep=None, chan_keep=None):
    """The reference kernel's attention dropout (attentions/attn.py:1052-1059, 222-227): whole key
    time steps and whole key channels are dropped, each with probability 1 - sqrt(1 - p_drop), the
    same keys for every sample, head and query; the probabilities of dropped keys are zeroed AFTER
    the soft-max sum and the others divided by 1 - p_drop.  The sum does not see the masks, so
    this is the plain attention on values v[k] * keep[k] / (1 - p_drop): returns that factor per
    key row [T*C] (fp32).  The masks are drawn as the reference draws them (channels first, then
    time steps, torch.rand(...) > p_per_dim on the device) unless they are given."""
    p_per_dim = 1.0 - (1.0 - p_drop) ** 0.5
    if chan_keep is None:
        chan_keep = torch.rand(chan_ctx, device=device, generator=generator) > p_per_dim
    if time_keep is None:
        time_keep = torch.rand(time_ctx, device=device, generator=generator) > p_per_dim
    keep = time_keep.to(device=device, dtype=torch.bool)[:, None] & chan_keep.to(device=device, dtype=torch.bool)[None, :]
    return keep.reshape(time_ctx * chan_ctx).to(torch.float32) / (1.0 - p_drop)


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
    time_keep=None,      # extension: the dropout's keep masks [T] / [C] given instead of drawn
    chan_keep=None,
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
        v = v * dropout_key_scale(p_drop, time_ctx, chan_ctx, q.device, generator,
                                  time_keep, chan_keep).to(v.dtype)[None, None, :, None]
    if window_size > 0 and not (rel_bias_chan or rel_bias_time):
        raise NotImplementedError(
            "flash_mvpa: a content window without relative biases (masking instead of zeroing) "
            "is not implemented")
    if not q.is_cuda:
        raise RuntimeError("flash_mvpa needs GPU tensors (there is no CPU path)")
    dh = q.shape[-1]
    if torch.is_grad_enabled() and any(
            t.requires_grad for t in (q, q_bias, q_btime, q_bchan, k_glob, k_time, k_chan, v)):
        if out is not None:
            raise NotImplementedError("flash_mvpa: a preallocated output cannot be used with autograd")
        return FlashMVPA.apply(
            q, q_bias.reshape(kv_heads, dh), q_btime.reshape(kv_heads, dh),
            q_bchan.reshape(kv_heads, dh), k_glob, k_time.reshape(kv_heads, time_ctx, dh),
            k_chan.reshape(kv_heads, chan_ctx, dh), v, bool(causal), sm_scale, int(window_size),
            bool(rel_bias_time), bool(rel_bias_chan), chan_valid)
    return mvpa_hip.mvpa_forward(
        q, k_glob, v,
        q_bias.reshape(kv_heads, dh), q_btime.reshape(kv_heads, dh), q_bchan.reshape(kv_heads, dh),
        k_time.reshape(kv_heads, time_ctx, dh), k_chan.reshape(kv_heads, chan_ctx, dh),
        sm_scale=sm_scale, window=int(window_size), causal=bool(causal), content=True,
        time_bias=bool(rel_bias_time), chan_bias=bool(rel_bias_chan), chan_valid=chan_valid,
        out=out, kernel=kernel)
