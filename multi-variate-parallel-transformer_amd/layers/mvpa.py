"""MVPA attention layers with the reference's module interface, running on the HIP kernels.

`MVPFormerGQAAttention` and `MVPFormerGQAFlashAttention` keep the constructor arguments,
parameter / buffer names, forward signature and return tuple of layers/mvpa.py:8-409, so a
model file written against the reference (models/mvpformer.py:104-152) can import them
unchanged and a reference state dict loads key for key.

What differs is mechanism only:
* q/k/v come out of ONE fused projection GEMM and are handed to the attention kernel as
  strided [B,T,C,H,Dh] views; the kernel writes its output already head-merged, so the
  permute+contiguous copies of _split_heads/_merge_heads (layers/mvpa.py:161-171) vanish.
* the score/softmax/PV chain of _rel_attn (layers/mvpa.py:173-278) is the fused kernel; no
  [B,H,N,N] tensor exists, hence `output_attentions=True` raises.
Forward / eval only (no autograd through the kernel).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

import mvpa_hip


class MvpaKVCache:
    """Keys and values of one layer for step-by-step decoding, kept in place.

    The `(k, v)` tuple of the reference's `layer_past` / `present` (layers/mvpa.py:314-321) grows
    by a concatenation per step, i.e. a copy of the whole cache.  This holder owns two buffers
    [B,Hkv,capacity,C,Dh] instead; a step writes its C new rows behind the cached ones and the
    attention kernel reads the live time steps through a strided view.  At most `max_steps` time
    steps are live (the new one included): once that many are cached the oldest drops out, which
    is the sliding window of a stream - the biases are relative, so the remaining steps keep their
    meaning.  The live steps move back to the front of the buffer once every `capacity -
    max_steps + 1` steps, so the copy is amortised.  Pass it wherever `layer_past` goes; the layer
    returns the same object as `present`."""

    def __init__(self, batch: int, kv_heads: int, channels: int, head_dim: int, max_steps: int,
                 dtype=torch.bfloat16, device="cuda", slack: Optional[int] = None):
        if max_steps < 1:
            raise ValueError("max_steps must be at least 1")
        slack = max(1, max_steps // 4) if slack is None else max(0, int(slack))
        self.max_steps = max_steps
        self.capacity = max_steps + slack
        self.k = torch.empty((batch, kv_heads, self.capacity, channels, head_dim), dtype=dtype, device=device)
        self.v = torch.empty_like(self.k)
        self.start = 0            # first live time step in the buffers
        self.length = 0           # live time steps

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """Add one time step ([B,Hkv,C,Dh] each); returns views [B,Hkv,T,C,Dh] of the live steps."""
        if self.length == self.max_steps:                 # the oldest step leaves the window
            self.start += 1
            self.length -= 1
        if self.start + self.length == self.capacity:     # out of room: live steps back to the front
            live_k = self.k[:, :, self.start:self.start + self.length].clone()
            live_v = self.v[:, :, self.start:self.start + self.length].clone()
            self.k[:, :, :self.length] = live_k
            self.v[:, :, :self.length] = live_v
            self.start = 0
        pos = self.start + self.length
        self.k[:, :, pos] = k_new
        self.v[:, :, pos] = v_new
        self.length += 1
        return self.views()

    def views(self) -> Tuple[torch.Tensor, torch.Tensor]:
        sl = slice(self.start, self.start + self.length)
        return self.k[:, :, sl], self.v[:, :, sl]

    def reset(self) -> None:
        self.start = self.length = 0


class MvpaRingClock:
    """The slot of the newest time step of one or several MvpaRingCaches, as a device counter (the
    attention kernel and the append kernel read it there).  The caches of all blocks of a stack
    move together, so they share one clock that advances once per step."""

    def __init__(self, steps: int, head: int, device):
        self.steps = steps
        self.head32 = torch.tensor([head], dtype=torch.int32, device=device)

    def advance(self) -> None:
        """On to the next slot (the oldest step's).  Device-side only: may run under graph capture."""
        self.head32.add_(1).remainder_(self.steps)


class MvpaRingCache:
    """A full window of keys and values as a ring: `steps` slots [B,Hkv,steps,C,Dh], the newest
    time step in slot `head` (a device counter), the one before it in slot head-1, and so on
    around the ring.  Appending overwrites the oldest slot, so nothing ever moves, every pointer
    stays where it is and the position of the newest step lives in device memory: one decoding step
    is then a fixed sequence of launches that a HIP graph can replay (MVPA_FLAG_RING tells the
    attention kernel which table row each slot stands for).  Always full: build it from a filled
    MvpaKVCache with `from_cache`.  With a clock of its own (the default) append() moves on to the
    next slot by itself; caches that share a clock write where the clock stands and whoever drives
    them advances it once per step."""

    def __init__(self, k: torch.Tensor, v: torch.Tensor, head: int = 0, clock: Optional[MvpaRingClock] = None):
        self.k, self.v = k.contiguous(), v.contiguous()      # [B,Hkv,steps,C,Dh]
        self.steps = k.shape[2]
        self.own_clock = clock is None
        self.clock = MvpaRingClock(self.steps, head, k.device) if clock is None else clock
        if self.clock.steps != self.steps:
            raise ValueError("clock and cache disagree on the number of slots")

    @property
    def head32(self) -> torch.Tensor:
        return self.clock.head32

    @classmethod
    def from_cache(cls, cache: "MvpaKVCache", clock: Optional[MvpaRingClock] = None) -> "MvpaRingCache":
        if cache.length != cache.max_steps:
            raise ValueError("the window is not full yet: keep appending to the MvpaKVCache")
        k, v = cache.views()
        return cls(k.clone(), v.clone(), cache.max_steps - 1, clock)   # time order: the newest step is last

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor) -> None:
        """One new time step ([B,Hkv,C,Dh] each) over the oldest slot.  Device-side only: may run
        under graph capture."""
        if self.own_clock:
            self.clock.advance()
        mvpa_hip.ring_append(k_new, v_new, self.k, self.v, self.clock.head32)


class KeyMask:
    """An additive key mask ([B,1,1,N], zeros and finfo.min: models/mvpformer.py:262-268) together
    with what the kernels make of it, worked out ONCE for all the layers that receive it.  A mask
    that is the same at every time step is a per-channel validity mask [B,C], which the bf16
    kernels apply exactly; anything else goes on as an additive key bias [B,N] (fp32 kernel).
    Built with chan_valid given, nothing is inspected and nothing synchronises with the device,
    so a forward with such a mask can be recorded into a graph."""

    def __init__(self, additive: Optional[torch.Tensor] = None, chan_valid: Optional[torch.Tensor] = None):
        if additive is None and chan_valid is None:
            raise ValueError("KeyMask needs the additive mask or the channel-validity mask")
        self.additive = additive
        self.chan_valid = chan_valid
        self._resolved = chan_valid is not None

    def resolve(self, bsz, t_len, c_len):
        if not self._resolved:
            self.chan_valid = MVPFormerGQAAttention._as_channel_validity(self.additive, bsz, t_len, c_len)
            self._resolved = True
        if self.chan_valid is not None:
            return self.chan_valid, None
        return None, self.additive.reshape(bsz, t_len * c_len).to(torch.float32)


class _LoRALinear(torch.nn.Linear):
    """Bias-free Linear with low-rank adapters under the parameter names the reference's
    adapter library uses (lora_A, lora_B; layers/mvpa.py:43-62, 86-93).  `enable` marks which
    equal slices of the output carry an adapter; the effective weight is
    W + (alpha/r) * B A on those slices.  lora_B is zero-initialised, so a fresh layer equals
    the plain Linear."""

    def __init__(self, in_features, out_features, r, lora_alpha, enable=(True,)):
        super().__init__(in_features, out_features, bias=False)
        self.r = r
        self.scaling = lora_alpha / r if r > 0 else 0.0
        self.enable = tuple(bool(e) for e in enable)
        n_on = sum(self.enable)
        if r > 0 and n_on > 0:
            self.lora_A = torch.nn.Parameter(self.weight.new_zeros((r * n_on, in_features)))
            self.lora_B = torch.nn.Parameter(
                self.weight.new_zeros((out_features // len(self.enable) * n_on, r)))
            torch.nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))

    def effective_weight(self) -> torch.Tensor:
        if self.r <= 0 or not hasattr(self, "lora_A"):
            return self.weight
        w = self.weight.clone()
        slice_rows = self.out_features // len(self.enable)
        j = 0
        for i, on in enumerate(self.enable):
            if on:
                a = self.lora_A[j * self.r:(j + 1) * self.r]
                b = self.lora_B[j * slice_rows:(j + 1) * slice_rows]
                w[i * slice_rows:(i + 1) * slice_rows] += (b @ a) * self.scaling
                j += 1
        return w

    def forward(self, x):
        return torch.nn.functional.linear(x, self.effective_weight())


def _weight_of(mod) -> torch.Tensor:
    return mod.effective_weight() if isinstance(mod, _LoRALinear) else mod.weight


def _linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """GPU tensors go through the library's MFMA GEMMs, bf16 or fp32."""
    if x.is_cuda and x.dtype == torch.bfloat16:
        return mvpa_hip.linear(x, w.to(torch.bfloat16))
    if x.is_cuda and x.dtype == torch.float32:
        return mvpa_hip.linear_f32(x, w.to(torch.float32))
    return torch.nn.functional.linear(x, w.to(x.dtype))


class MVPFormerGQAAttention(torch.nn.Module):
    """Interface of layers/mvpa.py:8-337."""

    # the flash subclass of the reference ignores attention_mask / head_mask
    # (layers/mvpa.py:341-397); this flag keeps that difference between the two classes
    _honours_masks = True
    _key_dropout = False       # attn_pdrop acts on the attention weights (layers/mvpa.py:273)

    def __init__(self, config, is_cross_attention=False, layer_idx=None):
        super().__init__()
        max_timesteps = config.max_position_embeddings
        self.register_buffer(
            "time_bias",
            torch.tril(torch.ones((max_timesteps, max_timesteps), dtype=torch.bool)).view(
                1, 1, max_timesteps, max_timesteps),
        )
        self.register_buffer("masked_bias", torch.tensor(-1e4))
        self.embed_dim = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.num_kv_heads = config.n_head_kv
        self.num_kv_groups = self.num_heads // self.num_kv_heads
        self.head_dim = self.embed_dim // self.num_heads
        self.embed_kv_dim = self.head_dim * self.num_kv_heads
        self.split_size = self.embed_dim
        self.inner_dim = config.n_inner
        self.global_att = config.global_att
        if self.head_dim * self.num_heads != self.embed_dim:
            raise ValueError(
                f"`embed_dim` must be divisible by num_heads (got `embed_dim`: {self.embed_dim} and "
                f"`num_heads`: {self.num_heads}).")
        self.scale_attn_weights = config.scale_attn_weights
        self.is_cross_attention = is_cross_attention
        self.scale_attn_by_inverse_layer_idx = config.scale_attn_by_inverse_layer_idx
        self.layer_idx = layer_idx
        self.reorder_and_upcast_attn = config.reorder_and_upcast_attn
        # extension: content-term QK^T in fp8 e4m3 with per-head amax scales (bf16 GPU path only)
        self.fp8_qk = bool(getattr(config, "fp8_qk", False))
        e, kv = self.embed_dim, self.embed_kv_dim
        if getattr(config, "lora", False):
            self.q_attn = _LoRALinear(e, e, config.lora_rank, config.lora_alpha, enable=(True,))
            self.c_attn = _LoRALinear(e, 2 * kv, config.lora_rank, config.lora_alpha,
                                      enable=(False, True))
        else:
            self.q_attn = torch.nn.Linear(e, e, bias=False)
            self.c_attn = torch.nn.Linear(e, 2 * kv, bias=False)
        self.position_net = torch.nn.Linear(e, kv, bias=False)
        self.channel_net = torch.nn.Linear(e, kv, bias=False)
        self.c_proj = torch.nn.Linear(e, e, bias=False)
        self.attn_bias = torch.nn.Parameter(torch.empty(3 * kv))
        torch.nn.init.normal_(self.attn_bias, std=0.02)
        self.attn_dropout = torch.nn.Dropout(config.attn_pdrop)
        self.resid_dropout = torch.nn.Dropout(config.resid_pdrop)
        self._fused_w = None
        self._fused_key = None
        self._tables = None
        self._tables_key = None

    def adapter_params(self):
        return ["q_attn.lora_A", "q_attn.lora_B", "c_attn.lora_A", "c_attn.lora_B"]

    # -- projections --------------------------------------------------------------------------
    def _qkv_weight(self, dtype) -> torch.Tensor:
        """[q_attn; c_attn] stacked once and cached until a weight is modified."""
        srcs = [self.q_attn.weight, self.c_attn.weight]
        for mod in (self.q_attn, self.c_attn):
            if isinstance(mod, _LoRALinear) and hasattr(mod, "lora_A"):
                srcs += [mod.lora_A, mod.lora_B]
        key = tuple((t.data_ptr(), t._version) for t in srcs) + (dtype,)
        if self._fused_key != key:
            self._fused_w = torch.cat([_weight_of(self.q_attn), _weight_of(self.c_attn)], 0).to(dtype).contiguous()
            self._fused_key = key
        return self._fused_w

    def _key_tables(self, positional_embedding, channel_embedding):
        """position_net(positional_embedding) -> [Hkv,T,Dh] and channel_net(channel_embedding) ->
        [Hkv,C,Dh] (layers/mvpa.py:307-313).  Both depend only on parameters and on the embedding
        rows, so they are computed once and reused until one of those tensors changes."""
        hkv, dh = self.num_kv_heads, self.head_dim
        t_len, c_len = positional_embedding.shape[-2], channel_embedding.shape[-2]

        def compute():
            k_time = _linear(positional_embedding, self.position_net.weight)
            k_chan = _linear(channel_embedding, self.channel_net.weight)
            return (k_time.view(t_len, hkv, dh).permute(1, 0, 2).contiguous(),
                    k_chan.view(c_len, hkv, dh).permute(1, 0, 2).contiguous())

        # only views of parameters can be recognised safely from one call to the next (their
        # version counter follows every in-place update); anything else is recomputed
        def ident(t):
            base = t._base if t._base is not None else t
            if not isinstance(base, torch.nn.Parameter):
                return None
            return (base.data_ptr(), base._version, t.storage_offset(), tuple(t.shape), tuple(t.stride()), t.dtype)

        ids = tuple(ident(t) for t in (positional_embedding, channel_embedding,
                                       self.position_net.weight, self.channel_net.weight))
        if any(i is None for i in ids):
            return compute()
        if self._tables_key != ids:
            self._tables, self._tables_key = compute(), ids
        return self._tables

    @staticmethod
    def _resolve_mask(attention_mask, bsz, t_len, c_len):
        """(chan_valid, key_bias) for the kernels.  A KeyMask was analysed by whoever made it (the
        stack does that once per forward, or is told the validity mask outright: no device
        synchronisation here); a plain additive tensor is analysed now."""
        if attention_mask is None:
            return None, None
        if isinstance(attention_mask, KeyMask):
            return attention_mask.resolve(bsz, t_len, c_len)
        return KeyMask(attention_mask).resolve(bsz, t_len, c_len)

    @staticmethod
    def _as_channel_validity(attention_mask, bsz, t_len, c_len):
        """An additive key mask built from a 0/1 mask (models/mvpformer.py:262-268: zeros and
        finfo.min) that is the same at every time step is a per-channel validity mask, which the
        bf16 MFMA kernel applies exactly.  Returns [B,C] bool, or None if the mask is anything else
        (then it is passed on as an additive key bias)."""
        m = attention_mask.reshape(bsz, t_len, c_len)
        first = m[:, 0]
        binary = ((first == 0) | (first <= -1e30)).all()
        same = (m == first[:, None]).all()
        if bool(binary & same):          # one device sync per call, only when a mask is given
            return first == 0
        return None

    def _scale(self) -> float:
        s = 1.0
        if self.scale_attn_weights:
            s /= self.head_dim ** 0.5                      # layers/mvpa.py:246-252
        if self.scale_attn_by_inverse_layer_idx:
            s /= float(self.layer_idx + 1)                 # layers/mvpa.py:253-254
        return s

    def _content(self) -> bool:
        return bool(self.global_att)                       # layers/mvpa.py:188-222, 230

    def _attend(self, hidden_states, positional_embedding, channel_embedding, attention_mask,
                head_mask, use_cache, window, layer_past=None, merged_out=None, qkv=None):
        """merged_out: a [B, T*C, H, Dh] view (unit last stride, any row pitch) that receives the
        merged heads; c_proj is then left to the caller and merged_out is what comes back.
        qkv: hidden_states @ [q_attn; c_attn]^T when the caller has already formed it."""
        if self.training and (self.attn_dropout.p > 0 or self.resid_dropout.p > 0):
            # dropout lives on the differentiable path (one launch per op); the fused inference
            # path has none
            if layer_past is not None or merged_out is not None or not torch.is_grad_enabled():
                raise NotImplementedError("MVPA HIP layer: dropout in train() mode goes with the "
                                          "whole-sequence forward in grad mode; call .eval() otherwise")
            if self.attn_dropout.p > 0 and not self._key_dropout:
                raise NotImplementedError(
                    "MVPA HIP layer: dropout on the [B,H,N,N] attention weights (layers/mvpa.py:273) "
                    "is not implemented - the weights are never formed; the flash layer's dropout "
                    "of whole key steps and channels (layers/mvpa.py:394) is")
        if self.is_cross_attention:
            raise NotImplementedError(
                "MVPA HIP layer: without the time-causal mask the relative-time shift of the "
                "reference reads wrapped entries (layers/mvpa.py:127-138); not supported")
        bsz, t_len, c_len, e = hidden_states.shape
        h, hkv, dh, kv = self.num_heads, self.num_kv_heads, self.head_dim, self.embed_kv_dim
        n = t_len * c_len
        dt = hidden_states.dtype
        if layer_past is not None:
            if merged_out is not None:
                raise NotImplementedError("merged_out goes with a whole-sequence forward")
            return self._attend_step(hidden_states, positional_embedding, channel_embedding,
                                     attention_mask, head_mask, use_cache, window, layer_past)
        if merged_out is None and qkv is None and self._wants_grad(hidden_states):
            return self._attend_autograd(hidden_states, positional_embedding, channel_embedding,
                                         attention_mask, head_mask, use_cache, window)
        with torch.no_grad():
            if qkv is None:
                qkv = _linear(hidden_states, self._qkv_weight(dt))      # [B,T,C,E+2kvE]
            row = e + 2 * kv
            qkv = qkv.view(bsz, n, row)
            q = qkv[:, :, :e].view(bsz, n, h, dh).permute(0, 2, 1, 3)        # views, no copy
            k = qkv[:, :, e:e + kv].view(bsz, n, hkv, dh).permute(0, 2, 1, 3)
            v = qkv[:, :, e + kv:].view(bsz, n, hkv, dh).permute(0, 2, 1, 3)
            k_time, k_chan = self._key_tables(positional_embedding, channel_embedding)
            u, vb, z = (b.view(hkv, dh) for b in self.attn_bias.split(kv, dim=0))
            chan_valid, key_bias = self._resolve_mask(attention_mask, bsz, t_len, c_len)
            merged = merged_out if merged_out is not None else \
                torch.empty((bsz, n, h, dh), dtype=dt, device=hidden_states.device)
            mvpa_hip.mvpa_forward(
                q, k, v, u, vb, z, k_time, k_chan, sm_scale=self._scale(), window=window,
                causal=True, content=self._content(), chan_valid=chan_valid,
                key_bias=key_bias, out=merged.permute(0, 2, 1, 3),
                fp8_qk=self.fp8_qk and dt == torch.bfloat16 and key_bias is None)
            if head_mask is not None:                       # layers/mvpa.py:274-275
                if head_mask.numel() != h:
                    raise NotImplementedError("head_mask must hold one factor per head")
                if merged_out is not None:
                    merged_out.mul_(head_mask.to(dt).reshape(1, 1, h, 1))
                else:
                    merged = merged * head_mask.to(dt).reshape(1, 1, h, 1)
            out = merged if merged_out is not None else \
                _linear(merged.view(bsz, t_len, c_len, e), self.c_proj.weight)
        present = None
        if use_cache is True:                               # layers/mvpa.py:318-321
            present = (k.reshape(bsz, hkv, t_len, c_len, dh), v.reshape(bsz, hkv, t_len, c_len, dh))
        return out, present

    def _wants_grad(self, hidden_states) -> bool:
        """Gradients are produced when grad mode is on and either the input carries a graph or the
        module is in train() mode (then for its parameters too); an eval() forward on a plain
        input stays on the fused inference path even outside torch.no_grad()."""
        return torch.is_grad_enabled() and (hidden_states.requires_grad or self.training)

    def _attend_autograd(self, hidden_states, positional_embedding, channel_embedding, attention_mask,
                         head_mask, use_cache, window):
        """The whole-sequence forward of layers/mvpa.py:280-337 as a differentiable graph: the four
        projections and c_proj through the library's GEMM (backward: two more GEMMs each), the
        attention through FlashMVPA (backward: mvpa_backward).  Same kernels as the inference path,
        launched one by one instead of fused."""
        from attentions.attn import FlashMVPA
        from mvpa_hip import autograd as AG
        bsz, t_len, c_len, e = hidden_states.shape
        h, hkv, dh, kv = self.num_heads, self.num_kv_heads, self.head_dim, self.embed_kv_dim
        n = t_len * c_len
        dt = hidden_states.dtype
        w_qkv = torch.cat([_weight_of(self.q_attn), _weight_of(self.c_attn)], 0)
        qkv = AG.linear(hidden_states, w_qkv).reshape(bsz, n, e + 2 * kv)
        q = qkv[:, :, :e].reshape(bsz, n, h, dh).permute(0, 2, 1, 3)
        k = qkv[:, :, e:e + kv].reshape(bsz, n, hkv, dh).permute(0, 2, 1, 3)
        v = v_plain = qkv[:, :, e + kv:].reshape(bsz, n, hkv, dh).permute(0, 2, 1, 3)
        k_time = AG.linear(positional_embedding, self.position_net.weight).reshape(t_len, hkv, dh).permute(1, 0, 2)
        k_chan = AG.linear(channel_embedding, self.channel_net.weight).reshape(c_len, hkv, dh).permute(1, 0, 2)
        u, vb, z = (b.reshape(hkv, dh).to(dt) for b in self.attn_bias.split(kv, dim=0))
        chan_valid, key_bias = self._resolve_mask(attention_mask, bsz, t_len, c_len)
        if self.training and self.attn_dropout.p > 0:
            # layers/mvpa.py:394: whole key steps and channels dropped, the rest scaled up; the
            # soft-max sum ignores the masks, so the values carry them (attentions.attn)
            from attentions.attn import dropout_key_scale
            v = v * dropout_key_scale(self.attn_dropout.p, t_len, c_len, v.device).to(dt)[None, None, :, None]
        out = FlashMVPA.apply(q, u, vb, z, k, k_time.contiguous(), k_chan.contiguous(), v, True,
                              self._scale(), window, True, True, chan_valid, self._content(), key_bias)
        merged = out.permute(0, 2, 1, 3)                                      # [B,N,H,Dh]
        if head_mask is not None:                                            # layers/mvpa.py:274-275
            if head_mask.numel() != h:
                raise NotImplementedError("head_mask must hold one factor per head")
            merged = merged * head_mask.to(dt).reshape(1, 1, h, 1)
        out = AG.linear(merged.reshape(bsz, t_len, c_len, e), self.c_proj.weight)
        out = self.resid_dropout(out)                                        # layers/mvpa.py:333, 401
        present = None
        if use_cache is True:
            present = (k.reshape(bsz, hkv, t_len, c_len, dh), v_plain.reshape(bsz, hkv, t_len, c_len, dh))
        return out, present

    def _attend_step(self, hidden_states, positional_embedding, channel_embedding, attention_mask,
                     head_mask, use_cache, window, layer_past):
        """One step of incremental decoding: hidden_states holds the new time step only
        ([B,1,C,E]), layer_past the keys and values of the steps before it ([B,Hkv,Tp,C,Dh] each,
        as returned in `present`, or an MvpaKVCache that is appended to in place),
        positional_embedding all Tp+1 positions.  The new keys and
        values are appended along the TIME axis; the reference's cache path concatenates along
        dim -2, the channel axis (layers/mvpa.py:314-317), which does not continue the sequence,
        and is not reproduced."""
        bsz, t_new, c_len, e = hidden_states.shape
        h, hkv, dh, kv = self.num_heads, self.num_kv_heads, self.head_dim, self.embed_kv_dim
        cache = layer_past if isinstance(layer_past, MvpaKVCache) else None
        ring = layer_past if isinstance(layer_past, MvpaRingCache) else None
        if ring is not None:
            t_past = ring.steps - 1
            past_k = ring.k
        elif cache is not None:
            t_past = min(cache.length, cache.max_steps - 1)
            past_k = cache.k
        else:
            past_k, past_v = layer_past
            t_past = past_k.shape[2]
        if t_new != 1:
            raise NotImplementedError("MVPA HIP layer: with layer_past, hidden_states holds one new time step")
        t_len = t_past + 1
        if positional_embedding.shape[-2] != t_len or past_k.shape[3] != c_len:
            raise ValueError("layer_past, positional_embedding and hidden_states disagree on T or C")
        dt = hidden_states.dtype
        with torch.no_grad():
            qkv = _linear(hidden_states, self._qkv_weight(dt)).view(bsz, c_len, e + 2 * kv)
            q = qkv[:, :, :e].view(bsz, c_len, h, dh).permute(0, 2, 1, 3)           # [B,H,C,Dh]
            k_new = qkv[:, :, e:e + kv].view(bsz, c_len, hkv, dh).permute(0, 2, 1, 3)
            v_new = qkv[:, :, e + kv:].view(bsz, c_len, hkv, dh).permute(0, 2, 1, 3)
            if ring is not None:
                if ring.k.dtype != dt:
                    raise ValueError("MvpaRingCache and hidden_states differ in dtype")
                ring.append(k_new, v_new)                                            # oldest slot overwritten
                k, v = ring.k, ring.v
            elif cache is not None:
                if cache.k.dtype != dt:
                    raise ValueError("MvpaKVCache and hidden_states differ in dtype")
                k, v = cache.append(k_new, v_new)                                    # views, in place
            else:
                k = torch.cat([past_k.to(dt), k_new.unsqueeze(2)], dim=2)            # [B,Hkv,T,C,Dh]
                v = torch.cat([past_v.to(dt), v_new.unsqueeze(2)], dim=2)
            k_time, k_chan = self._key_tables(positional_embedding, channel_embedding)
            u, vb, z = (b.view(hkv, dh) for b in self.attn_bias.split(kv, dim=0))
            chan_valid, key_bias = self._resolve_mask(attention_mask, bsz, t_len, c_len)
            merged = torch.empty((bsz, c_len, h, dh), dtype=dt, device=hidden_states.device)
            mvpa_hip.mvpa_forward(
                q, k.reshape(bsz, hkv, t_len * c_len, dh), v.reshape(bsz, hkv, t_len * c_len, dh),
                u, vb, z, k_time, k_chan, sm_scale=self._scale(), window=window, causal=True,
                content=self._content(), chan_valid=chan_valid, key_bias=key_bias,
                out=merged.permute(0, 2, 1, 3), last_step_only=True,
                ring_head=ring.head32 if ring is not None else None,
                fp8_qk=self.fp8_qk and dt == torch.bfloat16 and key_bias is None)
            if head_mask is not None:
                if head_mask.numel() != h:
                    raise NotImplementedError("head_mask must hold one factor per head")
                merged = merged * head_mask.to(dt).reshape(1, 1, h, 1)
            out = _linear(merged.view(bsz, 1, c_len, e), self.c_proj.weight)
        if ring is not None:
            return out, ring
        if cache is not None:
            return out, cache
        return out, ((k, v) if use_cache is True else None)

    def forward(
        self,
        hidden_states,
        positional_embedding,
        channel_embedding,
        layer_past: Optional[Tuple[torch.Tensor]] = None,
        attention_mask: Optional[torch.Tensor] = None,
        head_mask: Optional[torch.Tensor] = None,
        encoder_hidden_states: Optional[torch.Tensor] = None,
        encoder_attention_mask: Optional[torch.Tensor] = None,
        use_cache: Optional[bool] = False,
        output_attentions: Optional[bool] = False,
    ):
        if encoder_hidden_states is not None:
            raise NotImplementedError("MVPA HIP layer: cross attention is not implemented")
        if not self._honours_masks:
            attention_mask, head_mask = None, None
        elif output_attentions:
            raise NotImplementedError(
                "MVPA HIP layer: the fused kernel never forms the [B,H,N,N] attention weights")
        out, present = self._attend(hidden_states, positional_embedding, channel_embedding,
                                    attention_mask, head_mask, use_cache, window=10,
                                    layer_past=layer_past)
        outputs = (out, present)
        if output_attentions:
            outputs += (None,)                            # layers/mvpa.py:407-408
        return outputs


    def forward_merged(self, hidden_states, positional_embedding, channel_embedding, merged_out,
                       attention_mask=None, head_mask=None, use_cache=False, qkv=None):
        """forward() up to the merged heads: they are written into merged_out ([B, T*C, H, Dh], unit
        last stride, any row pitch) and c_proj (layers/mvpa.py:400) is left to the caller, who can
        fold it into a later product.  qkv: the fused q/kv projection of hidden_states
        (hidden_states @ qkv_weight()^T, contiguous) if the caller has formed it with another
        product.  Returns (merged_out, present)."""
        if not self._honours_masks:
            attention_mask, head_mask = None, None
        return self._attend(hidden_states, positional_embedding, channel_embedding, attention_mask,
                            head_mask, use_cache, window=10, merged_out=merged_out, qkv=qkv)

    def qkv_weight(self, dtype=torch.bfloat16) -> torch.Tensor:
        """[q_attn; c_attn] stacked (adapters folded in), cached until a weight changes."""
        return self._qkv_weight(dtype)


class MVPFormerGQAFlashAttention(MVPFormerGQAAttention):
    """Interface of layers/mvpa.py:340-409: same parameters, attention_mask / head_mask ignored,
    `None` in place of attention weights.  layer_past continues the sequence by one time step
    (see _attend_step)."""

    _honours_masks = False
    _key_dropout = True        # attn_pdrop drops whole key steps / channels inside the operator

    # The reference's flash layer calls its kernel with sm_scale = 1/sqrt(Dh) and the content term
    # always on, whatever scale_attn_weights, scale_attn_by_inverse_layer_idx and global_att say
    # (layers/mvpa.py:382-397); the same here, so the two classes differ exactly where the
    # reference's do.
    def _scale(self) -> float:
        return 1.0 / self.head_dim ** 0.5

    def _content(self) -> bool:
        return True

    def forward(self, hidden_states, positional_embedding, channel_embedding, layer_past=None,
                attention_mask=None, head_mask=None, encoder_hidden_states=None,
                encoder_attention_mask=None, use_cache=False, output_attentions=False):
        out, present = self._attend(hidden_states, positional_embedding, channel_embedding,
                                    None, None, use_cache, window=10, layer_past=layer_past)
        outputs = (out, present)
        if output_attentions:
            outputs += (None,)
        return outputs
