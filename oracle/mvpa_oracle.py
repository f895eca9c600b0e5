"""CPU oracle for MVPFormer's multi-variate parallel attention (MVPA) forward.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file; only the
tests, the smoke check and the benchmark's CPU-baseline leg do, and there only as the
checker / the reported baseline, never as the thing that is measured or shipped.

Three independent statements of the same operator live here:

* ``rel_attn``        - op-by-op restatement of the reference PyTorch path
                        (layers/mvpa.py:173-278), including the Transformer-XL style
                        pad-and-reshape shift (layers/mvpa.py:127-138) and the channel
                        gather (layers/mvpa.py:140-159).  Materialises [B,H,N,N].
* ``mvpa_direct``     - the closed form, evaluated per (b, h) and per query block so the
                        large configurations fit in RAM.  Indices are the closed forms
                        ``T-1-(tq-tk)`` and ``C-1-|cq-ck|`` that the reference's fused
                        kernel states a second time (attentions/attn.py:279-308).
* ``mvpa_bruteforce`` - pure-Python float64 loops straight from the definition, for tiny
                        inputs only.

Pinning status (what independent evidence fixes each function):
  rel_shift / rel_shift_chan : closed-form index maps on iota-coded tables (bit exact).
  rel_attn                   : torch SDPA special case (window vacuous, T <= 11);
                               float64 brute force (windowed, GQA, masks); invariants
                               (row-stochastic, causality, window locality, GQA == MHA).
  mvpa_direct                : equality with rel_attn on every small configuration.
  split_heads / merge_heads  : explicit index check, feature h*Dh+d of token (b,t,c) lands at
                               [b,h,t,c,d]; merge is the inverse (tests/test_oracle_stack.py).
  attention_layer_forward    : an einsum statement that never calls split/merge heads (named
                               head/dim axes, K = first half of c_attn, V = second) around the
                               float64 brute force; with and without the additive key mask; a
                               swapped K/V split is shown to fail (tests/test_oracle_stack.py).
  rmsnorm                    : torch.nn.functional.rms_norm and torch.nn.RMSNorm, fp32 and bf16,
                               plus a tiny-norm row that fixes eps inside the root.
  wave_encoder_forward       : torch.nn.RMSNorm + torch.nn.Linear around the pad + conv1d
                               statement of the wavelet transform.
  mvpformer_forward          : a composition of library modules (torch.nn.RMSNorm, Linear,
                               Embedding, transformers' LlamaMLP with mlp_bias=False) wired as
                               models/mvpformer.py:104-147, 246-283, 380 state it (parallel
                               block, both branches read ln_1(x), ln_2 unused, ln_f last), with
                               and without a token mask; a sequential block is shown to differ.
  wavedec_db4_periodic       : the reference delegates to ptwt.wavedec (ptwt==0.1.9 with
                               PyWavelets' db4 filters, models/fftencoder.py:62, 70-88), not
                               installed here.  Its published algorithm - circular pad of
                               (2*8-3)//2 = 6 samples left and 6 (+ n%2) right, one stride-2
                               conv1d with the flipped decomposition filters per level,
                               floor(log2(n/7)) levels, output [cA_L, cD_L .. cD_1] - is stated
                               a second time with torch's pad and conv1d in tests/test_oracle.py
                               and must agree for lengths 512, 2560 and odd lengths; the phase
                               is spelled out on unit impulses; plus the textbook properties
                               of the filter bank (orthogonality, energy, vanishing moments).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

# --------------------------------------------------------------------------------------
# head reshapes (layers/mvpa.py:161-171)
# --------------------------------------------------------------------------------------


def split_heads(x: torch.Tensor, num_heads: int, head_dim: int) -> torch.Tensor:
    """[B,T,C,H*Dh] -> [B,H,T,C,Dh]   (layers/mvpa.py:161-166)."""
    return x.view(x.shape[:-1] + (num_heads, head_dim)).permute(0, 3, 1, 2, 4)


def merge_heads(x: torch.Tensor, num_heads: int, head_dim: int) -> torch.Tensor:
    """[B,H,T,C,Dh] -> [B,T,C,H*Dh]   (layers/mvpa.py:168-171)."""
    x = x.permute(0, 2, 3, 1, 4).contiguous()
    return x.view(x.shape[:-2] + (num_heads * head_dim,))


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """GQA replication on dim 1 of a 5-D tensor (layers/mvpa.py:95-105)."""
    if n_rep == 1:
        return x
    b, hkv, a, c, d = x.shape
    return x[:, :, None].expand(b, hkv, n_rep, a, c, d).reshape(b, hkv * n_rep, a, c, d)


def repeat_channel(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[.., n, tlen] -> [.., n, tlen*n_rep], each column repeated n_rep times in place
    (layers/mvpa.py:107-115)."""
    if n_rep == 1:
        return x
    b, h, n, t = x.shape
    return x[:, :, :, :, None].expand(b, h, n, t, n_rep).reshape(b, h, n, t * n_rep)


def repeat_time(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[.., n, clen] -> [.., n, n_rep*clen], the whole row tiled n_rep times
    (layers/mvpa.py:117-125)."""
    if n_rep == 1:
        return x
    b, h, n, c = x.shape
    return x[:, :, :, None, :].expand(b, h, n, n_rep, c).reshape(b, h, n, n_rep * c)


# --------------------------------------------------------------------------------------
# the two relative shifts
# --------------------------------------------------------------------------------------


def rel_shift(x: torch.Tensor) -> torch.Tensor:
    """Pad-and-reshape shift of a [B,H,N,T] table (layers/mvpa.py:127-138).

    The tensor is re-viewed as [B,H,T,N], a zero column is prepended, the result is
    re-viewed as [B,H,N+1,T] and its first row dropped.  For key times tk <= tq this
    lands ``x[n, T-1-(tq-tk)]`` in column tk; columns tk > tq hold wrapped values.
    """
    b, h, n, t = x.shape
    pad = torch.zeros((b, h, t, 1), dtype=x.dtype, device=x.device)
    padded = torch.cat([pad, x.reshape(b, h, t, n)], dim=-1)
    padded = padded.reshape(b, h, n + 1, t)
    return padded[:, :, 1:, :].reshape(b, h, n, t)


def rel_shift_chan(x: torch.Tensor) -> torch.Tensor:
    """Channel gather of a [B,H,N,C] table (layers/mvpa.py:140-159):
    ``out[n, ck] = x[n, C-1-|cq-ck|]`` with ``cq = n % C``.

    The index matrix is built the way the reference builds it - the strictly upper
    triangle is filled row by row with 1, 2, ... and mirrored - rather than with an
    ``abs`` so that the test against the closed form compares two different statements.
    """
    c = x.shape[-1]
    n = x.shape[-2]
    dist = torch.zeros(c, c, dtype=torch.int64)
    for i in range(c - 1):
        run = torch.arange(1, c - i, dtype=torch.int64)
        dist[i, i + 1:] = run
        dist[i + 1:, i] = run
    idx = (c - 1 - dist).repeat(n // c, 1)
    rows = torch.arange(n).unsqueeze(1)
    return x[..., rows, idx]


# --------------------------------------------------------------------------------------
# op-by-op restatement of _rel_attn
# --------------------------------------------------------------------------------------


def rel_attn(
    query: torch.Tensor,          # [B,H,T,C,Dh]
    global_key: torch.Tensor,     # [B,Hkv,T,C,Dh]
    time_key: torch.Tensor,       # [1,Hkv,T,1,Dh]
    channel_key: torch.Tensor,    # [1,Hkv,1,C,Dh]
    value: torch.Tensor,          # [B,Hkv,T,C,Dh]
    attn_bias: torch.Tensor,      # [3*Hkv*Dh]  (u | v | z)
    *,
    global_att: bool = True,
    scale_attn_weights: bool = True,
    scale_attn_by_inverse_layer_idx: bool = False,
    layer_idx: Optional[int] = None,
    is_cross_attention: bool = False,
    attention_mask: Optional[torch.Tensor] = None,   # additive, broadcastable to [B,H,N,N]
    head_mask: Optional[torch.Tensor] = None,
    window: int = 10,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Follows layers/mvpa.py:173-278 line by line.  Returns (out [B,H,T,C,Dh],
    weights [B,H,N,N])."""
    bsz, num_heads, pos_len, chan_len, head_dim = query.shape
    num_kv = global_key.shape[1]
    groups = num_heads // num_kv
    tot_len = pos_len * chan_len
    kv_dim = num_kv * head_dim
    u, v, z = attn_bias.split(kv_dim, dim=0)                      # :185-187
    u = repeat_kv(split_heads(u[None, None, None, :], num_kv, head_dim), groups)
    v = repeat_kv(split_heads(v[None, None, None, :], num_kv, head_dim), groups)
    z = repeat_kv(split_heads(z[None, None, None, :], num_kv, head_dim), groups)
    time_k = repeat_kv(time_key, groups).squeeze(-2).transpose(-1, -2)      # [1,H,Dh,T]
    chan_k = repeat_kv(channel_key, groups).squeeze(-3).transpose(-1, -2)   # [1,H,Dh,C]
    time_q = (query + v).reshape(bsz, num_heads, -1, head_dim)              # :215-217
    chan_q = (query + z).reshape(bsz, num_heads, -1, head_dim)              # :218-220
    time_att = rel_shift(torch.matmul(time_q, time_k))                      # :223,225
    chan_att = rel_shift_chan(torch.matmul(chan_q, chan_k))                 # :224,226
    w = repeat_channel(time_att, chan_len) + repeat_time(chan_att, pos_len)  # :227-229
    if global_att:
        glob_k = repeat_kv(global_key, groups).reshape(
            bsz, num_heads, tot_len, head_dim).transpose(-1, -2)
        glob_q = (query + u).reshape(bsz, num_heads, -1, head_dim)
        content = torch.matmul(glob_q, glob_k)                              # :222
        ones = torch.ones((pos_len, pos_len), dtype=torch.bool)
        win = torch.logical_and(torch.tril(ones, diagonal=window),
                                torch.triu(ones, diagonal=-window))          # :231-240
        win = win.repeat_interleave(chan_len, 0).repeat_interleave(chan_len, 1)
        win[-chan_len:] = True                                              # :244
        w = w + content.masked_fill(~win, 0.0)                              # :245
    if scale_attn_weights:
        w = w / torch.full([], head_dim ** 0.5, dtype=w.dtype)              # :246-252
    if scale_attn_by_inverse_layer_idx:
        w = w / float(layer_idx + 1)                                        # :253-254
    if not is_cross_attention:
        causal = torch.tril(torch.ones((pos_len, pos_len), dtype=torch.bool))
        causal = causal.repeat_interleave(chan_len, 0).repeat_interleave(chan_len, 1)
        w = w.masked_fill(~causal, torch.finfo(w.dtype).min)                # :255-264
    if attention_mask is not None:
        w = w + attention_mask                                              # :265-266
    if value.dtype == torch.float16:
        w = torch.softmax(w, dim=-1, dtype=torch.bfloat16).to(value.dtype)  # :267-270
    else:
        w = torch.softmax(w, dim=-1)                                        # :272
    if head_mask is not None:
        w = w * head_mask                                                   # :274-275
    val = repeat_kv(value, groups)
    out = torch.matmul(w, val.flatten(2, 3))                                # :277
    return out.view_as(val), w


def attention_layer_forward(
    hidden: torch.Tensor,          # [B,T,C,E]
    pos_emb: torch.Tensor,         # [1,T,E]
    chan_emb: torch.Tensor,        # [1,C,E]
    weights: dict,                 # q_attn.weight, c_attn.weight, position_net.weight,
                                   # channel_net.weight, c_proj.weight, attn_bias
    num_heads: int,
    num_kv_heads: int,
    attention_mask: Optional[torch.Tensor] = None,
    **flags,
) -> torch.Tensor:
    """MVPFormerGQAAttention.forward in eval mode (layers/mvpa.py:280-337)."""
    lin = torch.nn.functional.linear
    e = hidden.shape[-1]
    dh = e // num_heads
    kv_dim = dh * num_kv_heads
    q = lin(hidden, weights["q_attn.weight"])
    k, v = lin(hidden, weights["c_attn.weight"]).split(kv_dim, dim=-1)
    tk = lin(pos_emb, weights["position_net.weight"]).unsqueeze(2)
    ck = lin(chan_emb, weights["channel_net.weight"]).unsqueeze(1)
    q = split_heads(q, num_heads, dh)
    k = split_heads(k, num_kv_heads, dh)
    v = split_heads(v, num_kv_heads, dh)
    tk = split_heads(tk, num_kv_heads, dh)
    ck = split_heads(ck, num_kv_heads, dh)
    out, _ = rel_attn(q, k, tk, ck, v, weights["attn_bias"],
                      attention_mask=attention_mask, **flags)
    out = merge_heads(out, num_heads, dh)
    return lin(out, weights["c_proj.weight"])


# --------------------------------------------------------------------------------------
# closed form, chunked (fits the large configurations)
# --------------------------------------------------------------------------------------


def time_index(tq: torch.Tensor, tk: torch.Tensor, t_len: int) -> torch.Tensor:
    """Row of the time table used by query time tq for key time tk (valid for tk<=tq)."""
    return t_len - 1 - (tq - tk)


def chan_index(cq: torch.Tensor, ck: torch.Tensor, c_len: int) -> torch.Tensor:
    return c_len - 1 - (cq - ck).abs()


def window_active(tq: torch.Tensor, tk: torch.Tensor, t_len: int, window: int) -> torch.Tensor:
    """Content term is kept iff |tq-tk| <= window or tq is the last time step
    (layers/mvpa.py:231-245); window <= 0 keeps it everywhere."""
    if window <= 0:
        return torch.ones(torch.broadcast_shapes(tq.shape, tk.shape), dtype=torch.bool)
    return ((tq - tk).abs() <= window) | (tq == t_len - 1)


def mvpa_direct(
    q: torch.Tensor,        # [B,H,N,Dh]
    k: torch.Tensor,        # [B,Hkv,N,Dh]
    v: torch.Tensor,        # [B,Hkv,N,Dh]
    u: torch.Tensor,        # [Hkv,Dh] content bias
    vb: torch.Tensor,       # [Hkv,Dh] time bias
    z: torch.Tensor,        # [Hkv,Dh] channel bias
    k_time: torch.Tensor,   # [Hkv,T,Dh]
    k_chan: torch.Tensor,   # [Hkv,C,Dh]
    *,
    sm_scale: Optional[float] = None,
    window: int = 10,
    global_att: bool = True,
    chan_valid: Optional[torch.Tensor] = None,   # [B,C] bool
    key_bias: Optional[torch.Tensor] = None,     # [B,N] additive (already in score units)
    dtype: torch.dtype = torch.float64,
    q_block: int = 2048,
    heads: Optional[list] = None,                # subset of (b, h) pairs to evaluate
    q_ranges: Optional[list] = None,             # subset of query rows: [(n0, n1), ...]
    return_lse: bool = False,
):
    """Closed-form MVPA: score = s*[W*(q+u).k + (q+v).r[T-1-(tq-tk)] + (q+z).e[C-1-|cq-ck|]],
    time-causal mask, softmax over keys, times V.  Evaluated in ``dtype`` per (b,h) and
    per block of ``q_block`` queries.  Returns out [B,H,N,Dh] (rows of heads not listed
    in ``heads`` are left zero) and optionally the base-2 log-sum-exp [B,H,N]."""
    bsz, nh, n, dh = q.shape
    hkv = k.shape[1]
    t_len, c_len = k_time.shape[1], k_chan.shape[1]
    assert n == t_len * c_len
    grp = nh // hkv
    s = (1.0 / math.sqrt(dh)) if sm_scale is None else sm_scale
    out = torch.zeros((bsz, nh, n, dh), dtype=dtype)
    lse = torch.zeros((bsz, nh, n), dtype=dtype)
    pairs = heads if heads is not None else [(b, h) for b in range(bsz) for h in range(nh)]
    n_idx = torch.arange(n)
    tk_all, ck_all = n_idx // c_len, n_idx % c_len
    neg = torch.finfo(dtype).min
    for (b, h) in pairs:
        g = h // grp
        kk = k[b, g].to(dtype)
        vv = v[b, g].to(dtype)
        r = k_time[g].to(dtype)
        e = k_chan[g].to(dtype)
        blocks = []
        for (r0, r1) in (q_ranges if q_ranges is not None else [(0, n)]):
            blocks += [(x, min(r1, x + q_block)) for x in range(r0, r1, q_block)]
        for (q0, q1) in blocks:
            qq = q[b, h, q0:q1].to(dtype)
            tq = (n_idx[q0:q1] // c_len)[:, None]
            cq = (n_idx[q0:q1] % c_len)[:, None]
            hi = int(tq.max().item() + 1) * c_len     # keys past this are causally masked
            tk, ck = tk_all[None, :hi], ck_all[None, :hi]
            st = (qq + vb[g].to(dtype)) @ r.T                     # [m,T]
            sc = (qq + z[g].to(dtype)) @ e.T                      # [m,C]
            ti = time_index(tq, tk, t_len).clamp_(0, t_len - 1)
            ci = chan_index(cq, ck, c_len)
            score = torch.gather(st, 1, ti) + torch.gather(sc, 1, ci)
            if global_att:
                content = (qq + u[g].to(dtype)) @ kk[:hi].T
                score = score + content * window_active(tq, tk, t_len, window)
            score = score * s
            score = score.masked_fill(tk > tq, neg)
            if key_bias is not None:
                score = score + key_bias[b, :hi].to(dtype)[None, :]
            if chan_valid is not None:
                score = score + (~chan_valid[b])[ck_all[:hi]].to(dtype)[None, :] * neg
            m = score.max(dim=1, keepdim=True).values
            p = torch.exp(score - m)
            l = p.sum(dim=1, keepdim=True)
            out[b, h, q0:q1] = (p @ vv[:hi]) / l
            lse[b, h, q0:q1] = ((m + torch.log(l)) * math.log2(math.e)).squeeze(1)
    if return_lse:
        return out, lse
    return out


def mvpa_bruteforce(q, k, v, u, vb, z, k_time, k_chan, *, sm_scale=None, window=10,
                    global_att=True, chan_valid=None):
    """Float64 Python loops from the definition.  Tiny inputs only."""
    bsz, nh, n, dh = q.shape
    hkv = k.shape[1]
    t_len, c_len = k_time.shape[1], k_chan.shape[1]
    grp = nh // hkv
    s = (1.0 / math.sqrt(dh)) if sm_scale is None else sm_scale
    q, k, v, u, vb, z, k_time, k_chan = [x.double().tolist() for x in (q, k, v, u, vb, z, k_time, k_chan)]
    out = torch.zeros((bsz, nh, n, dh), dtype=torch.float64)

    def dot(a, bias, c):
        return sum((a[d] + bias[d]) * c[d] for d in range(dh))

    for b in range(bsz):
        for h in range(nh):
            g = h // grp
            for nq in range(n):
                tq, cq = divmod(nq, c_len)
                scores, keys = [], []
                for nk in range(n):
                    tk, ck = divmod(nk, c_len)
                    if tk > tq:
                        continue
                    if chan_valid is not None and not bool(chan_valid[b][ck]):
                        continue
                    sc = dot(q[b][h][nq], vb[g], k_time[g][t_len - 1 - (tq - tk)])
                    sc += dot(q[b][h][nq], z[g], k_chan[g][c_len - 1 - abs(cq - ck)])
                    if global_att and (window <= 0 or tq - tk <= window or tq == t_len - 1):
                        sc += dot(q[b][h][nq], u[g], k[b][g][nk])
                    scores.append(sc * s)
                    keys.append(nk)
                m = max(scores)
                ps = [math.exp(x - m) for x in scores]
                l = sum(ps)
                for d in range(dh):
                    out[b, h, nq, d] = sum(p * v[b][g][nk][d] for p, nk in zip(ps, keys)) / l
    return out


# --------------------------------------------------------------------------------------
# segment encoder (models/fftencoder.py:49-106)
# --------------------------------------------------------------------------------------

DB4_DEC_LO = [
    -0.010597401784997278, 0.032883011666982945, 0.030841381835986965, -0.18703481171888114,
    -0.02798376941698385, 0.6308807679295904, 0.7148465705525415, 0.23037781330885523,
]
DB4_DEC_HI = [((-1.0) ** (i + 1)) * DB4_DEC_LO[7 - i] for i in range(8)]


def dwt_max_level(n: int, filt_len: int = 8) -> int:
    """floor(log2(n / (filt_len-1))) - the rule the wavelet library applies
    (call site models/fftencoder.py:71)."""
    return max(0, int(math.floor(math.log2(n / (filt_len - 1)))))


def dwt_coeff_len_periodic(n: int, filt_len: int = 8) -> int:
    """Coefficient length for the "periodic" extension mode: floor((n+filt_len-1)/2)
    (call site models/fftencoder.py:74)."""
    return (n + filt_len - 1) // 2


def dwt_sizes(size_input: int):
    """models/fftencoder.py:70-78: sizes of every detail level then the last size again
    for the approximation; their sum is the projection's input width."""
    sizes, n = [], size_input
    for _ in range(dwt_max_level(size_input)):
        n = dwt_coeff_len_periodic(n)
        sizes.append(n)
    sizes.append(n)
    return sizes


def dwt_level_periodic(a: torch.Tensor):
    """One analysis level with periodic extension:
    out[k] = sum_j filt[j] * a[(2k+1-j) mod n],  k in [0, floor((n+7)/2))."""
    n = a.shape[-1]
    m = dwt_coeff_len_periodic(n)
    kk = torch.arange(m)[:, None]
    jj = torch.arange(8)[None, :]
    idx = (2 * kk + 1 - jj) % n
    taps = a[..., idx]                                            # [..., m, 8]
    lo = torch.tensor(DB4_DEC_LO, dtype=a.dtype)
    hi = torch.tensor(DB4_DEC_HI, dtype=a.dtype)
    return taps @ lo, taps @ hi


def wavedec_db4_periodic(x: torch.Tensor) -> torch.Tensor:
    """Multilevel db4 analysis, coefficients concatenated [cA_L, cD_L, ..., cD_1]
    (models/fftencoder.py:80-88)."""
    a = x.to(torch.float32)
    details = []
    for _ in range(dwt_max_level(x.shape[-1])):
        a, d = dwt_level_periodic(a)
        details.append(d)
    return torch.cat([a] + details[::-1], dim=-1)


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(x.dtype)


def wave_encoder_forward(x: torch.Tensor, ln_weight: torch.Tensor, proj_weight: torch.Tensor):
    """WaveEncoder.forward (models/fftencoder.py:90-97)."""
    y = rmsnorm(wavedec_db4_periodic(x), ln_weight, 1e-5)
    return torch.nn.functional.linear(y.to(x.dtype), proj_weight)


# --------------------------------------------------------------------------------------
# model stack (models/mvpformer.py:104-152, 190-402, 596-607)
# --------------------------------------------------------------------------------------


def mvpformer_forward(x: torch.Tensor, params: dict, cfg: dict,
                      attention_mask: Optional[torch.Tensor] = None):
    """Encoder -> n_layer parallel blocks -> final norm, eval mode.

    ``x`` is [B,T,C,L] raw segments.  ``params`` uses the reference state-dict names
    (encoder.ln.weight, encoder.proj.weight, mvpformer.h.{i}.ln_1.weight,
    mvpformer.h.{i}.attn.*, mvpformer.h.{i}.mlp.{gate,up,down}_proj.weight,
    mvpformer.ln_f.weight, mvpformer.positional_embedding.weight,
    mvpformer.channel_embedding.weight).  Returns (out [B,T,C,E], embeds [B,T,C,E]).
    """
    lin = torch.nn.functional.linear
    b, t, c, seg = x.shape
    enc = wave_encoder_forward(x.reshape(b * t * c, seg), params["encoder.ln.weight"],
                               params["encoder.proj.weight"])
    embeds = enc.view(b, t, c, -1)                                  # mvpformer.py:599-604
    pos = params["mvpformer.positional_embedding.weight"][:t][None]  # :246-253, 282
    chan = params["mvpformer.channel_embedding.weight"][:c][None]    # :254-261, 283
    am = None
    if attention_mask is not None:                                  # :262-268
        am = attention_mask.view(b, -1)[:, None, None, :].to(embeds.dtype)
        am = (1.0 - am) * torch.finfo(embeds.dtype).min
    eps = cfg.get("layer_norm_epsilon", 1e-5)
    h = embeds
    for i in range(cfg["n_layer"]):
        pre = f"mvpformer.h.{i}."
        hn = rmsnorm(h, params[pre + "ln_1.weight"], eps)           # :133
        attn_w = {kk[len(pre + "attn."):]: vv for kk, vv in params.items()
                  if kk.startswith(pre + "attn.")}
        a = attention_layer_forward(hn, pos, chan, attn_w, cfg["n_head"], cfg["n_head_kv"],
                                    attention_mask=am)               # :134-143
        gate = lin(hn, params[pre + "mlp.gate_proj.weight"])
        up = lin(hn, params[pre + "mlp.up_proj.weight"])
        mlp = lin(torch.nn.functional.silu(gate) * up, params[pre + "mlp.down_proj.weight"])
        h = h + mlp + a                                             # :146-147
    h = rmsnorm(h, params["mvpformer.ln_f.weight"], eps)            # :380
    return h, embeds
