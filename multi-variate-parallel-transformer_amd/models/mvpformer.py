"""MVPFormer stack on the HIP library: config, parallel block, model, head and the inference
wrapper, with the reference's class names, constructor arguments and state-dict keys
(models/mvpformer.py:37-152, 155-402, 405-479, 596-607, 979-989) but without the training
harness (no Lightning, no HF base classes).  bf16 on the GPU.

Two paths through every module.  Inference (eval() mode, or under torch.no_grad()): fused
launches, nothing kept for a backward.  Differentiable (grad mode on and either train() mode or
an input that carries a graph): the same kernels one product at a time through
mvpa_hip.autograd and attentions.attn.FlashMVPA, so that gradients reach the input and every
parameter as they do through models/mvpformer.py:132-147 and layers/mvpa.py:280-337.  Dropout
(embd_pdrop, resid_pdrop, and attn_pdrop as the flash layer applies it) acts on that path only.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

import mvpa_hip
from mvpa_hip import autograd as AG
from layers import (KeyMask, MvpaKVCache, MvpaRingCache, MvpaRingClock, MVPFormerGQAAttention,
                    MVPFormerGQAFlashAttention)
from models import BrainDecider, BrainEncoder, BrainModel
from models.fftencoder import RMSNorm


class MVPFormerConfig:
    """Same constructor arguments and attribute aliases as models/mvpformer.py:37-101."""

    attribute_map = {
        "hidden_size": "n_embd",
        "max_position_embeddings": "n_positions",
        "max_channel_embeddings": "n_channels",
        "num_attention_heads": "n_head",
        "num_hidden_layers": "n_layer",
        "intermediate_size": "n_inner",
        "hidden_act": "activation_function",
    }

    def __init__(self, n_positions=100, n_channels=128, n_embd=768, n_layer=12, n_head=12,
                 n_inner=2048, n_head_kv=12, global_att=True, activation_function="silu",
                 resid_pdrop=0.1, embd_pdrop=0.1, attn_pdrop=0.1, layer_norm_epsilon=0.00001,
                 initializer_range=0.02, scale_attn_weights=True, use_cache=False,
                 scale_attn_by_inverse_layer_idx=False, reorder_and_upcast_attn=False,
                 lora=False, lora_alpha=16, lora_rank=8, lora_dropout=0, lora_merge=True,
                 fp8_qk=False):
        self.n_positions, self.n_channels, self.n_embd = n_positions, n_channels, n_embd
        self.n_layer, self.n_head, self.n_inner, self.n_head_kv = n_layer, n_head, n_inner, n_head_kv
        self.global_att = global_att
        self.activation_function = activation_function
        self.resid_pdrop, self.embd_pdrop, self.attn_pdrop = resid_pdrop, embd_pdrop, attn_pdrop
        self.layer_norm_epsilon = layer_norm_epsilon
        self.initializer_range = initializer_range
        self.scale_attn_weights = scale_attn_weights
        self.use_cache = use_cache
        self.scale_attn_by_inverse_layer_idx = scale_attn_by_inverse_layer_idx
        self.reorder_and_upcast_attn = reorder_and_upcast_attn
        self.pretraining_tp = 1
        self.mlp_bias = False
        self.lora, self.lora_alpha, self.lora_rank = lora, lora_alpha, lora_rank
        self.lora_dropout, self.lora_merge = lora_dropout, lora_merge
        self.fp8_qk = fp8_qk            # extension: fp8 e4m3 QK^T of the content term
        self.add_cross_attention = False
        self.output_attentions = False
        self.output_hidden_states = False

    def __getattr__(self, name):
        amap = type(self).attribute_map
        if name in amap:
            return getattr(self, amap[name])
        raise AttributeError(name)

    @classmethod
    def from_yaml(cls, path: str) -> "MVPFormerConfig":
        """Read the gpt_config block of one of the reference's YAML files (configs/*.yaml:49-71)."""
        import yaml
        with open(path) as f:
            doc = yaml.safe_load(f)
        return cls(**doc["model"]["init_args"]["gpt_config"]["init_args"])


class GatedMLP(nn.Module):
    """down(silu(gate(x)) * up(x)), bias-free: the MLP the reference takes from the Llama family
    (models/mvpformer.py:114).  gate and up run as ONE GEMM with the SiLU-multiply fused."""

    def __init__(self, config):
        super().__init__()
        h, m = config.hidden_size, config.intermediate_size
        self.gate_proj = nn.Linear(h, m, bias=False)
        self.up_proj = nn.Linear(h, m, bias=False)
        self.down_proj = nn.Linear(m, h, bias=False)
        self._gu = None
        self._gu_key = None

    def _gate_up(self) -> torch.Tensor:
        key = (self.gate_proj.weight.data_ptr(), self.gate_proj.weight._version,
               self.up_proj.weight.data_ptr(), self.up_proj.weight._version)
        if self._gu_key != key:
            self._gu = torch.cat([self.gate_proj.weight, self.up_proj.weight], 0).detach().to(torch.bfloat16).contiguous()
            self._gu_key = key
        return self._gu

    def forward(self, x):
        if torch.is_grad_enabled() and (x.requires_grad or self.training):
            mid = torch.nn.functional.silu(AG.linear(x, self.gate_proj.weight)) * AG.linear(x, self.up_proj.weight)
            return AG.linear(mid, self.down_proj.weight)
        with torch.no_grad():
            mid = mvpa_hip.linear(x, self._gate_up(), gated=True)
            return mvpa_hip.linear(mid, self.down_proj.weight.to(torch.bfloat16))

    def gate_up_weight(self) -> torch.Tensor:
        """[gate_proj; up_proj] stacked in bf16, cached until a weight changes."""
        return self._gate_up()

    @torch.no_grad()
    def activations_into(self, x, out):
        """silu(gate(x)) * up(x) written into out, a [rows, intermediate] view of any row pitch:
        the MLP up to its down projection, for a caller that folds that into a later product."""
        mvpa_hip.linear(x, self._gate_up(), gated=True, out=out)


class MVPFormerBlock(nn.Module):
    """Parallel block: x + MLP(ln_1(x)) + Attn(ln_1(x)); ln_2 exists but is unused
    (models/mvpformer.py:104-152)."""

    def __init__(self, config, layer_idx=None, flash: bool = True):
        super().__init__()
        hidden_size = config.hidden_size
        self.ln_1 = RMSNorm(hidden_size, eps=config.layer_norm_epsilon)
        cls = MVPFormerGQAFlashAttention if flash else MVPFormerGQAAttention
        self.attn = cls(config, layer_idx=layer_idx)
        self.ln_2 = RMSNorm(hidden_size, eps=config.layer_norm_epsilon)
        self.mlp = GatedMLP(config)
        self._tail_w = None
        self._tail_key = None
        self._fold_w = None
        self._fold_key = None

    def _tail_weight(self) -> torch.Tensor:
        """[c_proj | down_proj] side by side ([E, E + intermediate]), cached until one changes:
        attn_out + mlp_out = [merged heads | MLP activations] @ this^T."""
        wc, wd = self.attn.c_proj.weight, self.mlp.down_proj.weight
        key = (wc.data_ptr(), wc._version, wd.data_ptr(), wd._version)
        if self._tail_key != key:
            self._tail_w = torch.cat([wc, wd], 1).detach().to(torch.bfloat16).contiguous()
            self._tail_key = key
        return self._tail_w

    def _folded_weights(self):
        """[q_attn; c_attn] and [gate; up] with ln_1's weight folded into their columns
        (w[n][k] * ln_1[k], formed in fp32, rounded to bf16), cached until a source changes: the
        operands of the products that apply ln_1 in their epilogue (forward_norm_fused)."""
        wq, wg, ln = self.attn.qkv_weight(), self.mlp.gate_up_weight(), self.ln_1.weight
        key = (wq.data_ptr(), wq._version, wg.data_ptr(), wg._version, ln.data_ptr(), ln._version)
        if self._fold_key != key:
            scale = ln.detach().float()[None, :]
            self._fold_w = ((wq.float() * scale).to(torch.bfloat16).contiguous(),
                            (wg.float() * scale).to(torch.bfloat16).contiguous())
            self._fold_key = key
        return self._fold_w

    def norm_fused_supported(self, rows: int) -> bool:
        e, inner = self.attn.embed_dim, self.mlp.down_proj.in_features
        return (mvpa_hip.linear_dual_supported(rows, e) and mvpa_hip.linear_norm_fused_supported(rows, e + inner, e)
                and mvpa_hip.linear_residual_supported(rows, e + inner))

    @torch.no_grad()
    def forward_norm_fused(self, hidden_states, sumsq, positional_embedding, channel_embedding,
                           attention_mask=None, use_cache=False, both=None):
        """The block on its RAW input, ln_1 applied inside the products (models/mvpformer.py:133):
        `sumsq` holds the partial sums of squares of hidden_states' rows, as the previous block's
        tail product (or mvpa_hip.row_sumsq) wrote them; the q/kv and gate/up products multiply
        the raw rows with weights that carry ln_1's weight and scale each output row by its
        rsqrt(mean square + eps) in the epilogue; the tail product writes the next block's
        statistics beside its rows.  No norm kernel runs.  `both`: a [rows, E + intermediate]
        bf16 scratch buffer to reuse.  Returns (outputs, sumsq of the output rows)."""
        bsz, t_len, c_len, e = hidden_states.shape
        inner = self.mlp.down_proj.in_features
        rows = bsz * t_len * c_len
        h, dh = self.attn.num_heads, self.attn.head_dim
        if both is None:
            both = torch.empty((rows, e + inner), dtype=torch.bfloat16, device=hidden_states.device)
        merged = both[:, :e].unflatten(0, (bsz, t_len * c_len)).unflatten(2, (h, dh))
        wq, wg = self._folded_weights()
        x2 = hidden_states.reshape(rows, e)
        qkv, _ = mvpa_hip.linear_dual(x2, wq, wg, out_gated=both[:, e:], sumsq=sumsq, eps=self.ln_1.eps)
        _, present = self.attn.forward_merged(hidden_states, positional_embedding, channel_embedding, merged,
                                              attention_mask=attention_mask, use_cache=use_cache, qkv=qkv)
        out, sumsq = mvpa_hip.linear(both, self._tail_weight(), residual=x2, sumsq_out=True)
        out = out.view(hidden_states.shape)
        return ((out, present) if use_cache else (out,)), sumsq

    def forward(self, hidden_states, positional_embedding, channel_embedding, layer_past=None,
                attention_mask=None, head_mask=None, encoder_hidden_states=None,
                encoder_attention_mask=None, use_cache=False, output_attentions=False):
        outputs, _ = self.forward_fused(hidden_states, None, None, positional_embedding,
                                        channel_embedding, layer_past=layer_past,
                                        attention_mask=attention_mask, head_mask=head_mask,
                                        use_cache=use_cache, output_attentions=output_attentions)
        return outputs

    def forward_fused(self, hidden_states, normed, next_norm, positional_embedding,
                      channel_embedding, layer_past=None, attention_mask=None, head_mask=None,
                      use_cache=False, output_attentions=False):
        """The block with its norms at the seams: `normed` is ln_1(hidden_states) when the caller
        already has it, `next_norm` the RMSNorm that will consume this block's output (the next
        block's ln_1, or ln_f).  Returns (outputs, next_norm(output) or None); the residual sum and
        that norm come out of one kernel."""
        if layer_past is None and torch.is_grad_enabled() and (hidden_states.requires_grad or self.training):
            # differentiable path (models/mvpformer.py:132-147 op by op; both branches read ln_1(x))
            if normed is None:
                normed = self.ln_1(hidden_states)
            attn_outputs = self.attn(normed, positional_embedding, channel_embedding,
                                     attention_mask=attention_mask, head_mask=head_mask,
                                     use_cache=use_cache, output_attentions=output_attentions)
            hidden_states = hidden_states + self.mlp(normed) + attn_outputs[0]
            outputs = (hidden_states,) + (attn_outputs[1:] if use_cache else attn_outputs[2:])
            return outputs, (next_norm(hidden_states) if next_norm is not None else None)
        residual = hidden_states
        if normed is None:
            normed = self.ln_1(hidden_states)
        e, inner = self.attn.embed_dim, self.mlp.down_proj.in_features
        rows = hidden_states.numel() // e
        if (layer_past is None and not output_attentions and residual.is_cuda
                and residual.dtype == torch.bfloat16 and normed.dtype == torch.bfloat16
                and (head_mask is None or not self.attn._honours_masks)
                and mvpa_hip.linear_residual_supported(rows, e + inner)):
            # One product for the whole tail of the block: the attention kernel writes the merged
            # heads and the gate/up product its activations side by side into one buffer, and
            # hidden + c_proj(merged) + down(activations) = hidden + [merged | act] @ [c_proj | down]^T
            bsz, t_len, c_len, _ = hidden_states.shape
            h, dh = self.attn.num_heads, self.attn.head_dim
            both = torch.empty((rows, e + inner), dtype=torch.bfloat16, device=residual.device)
            merged = both[:, :e].unflatten(0, (bsz, t_len * c_len)).unflatten(2, (h, dh))
            if mvpa_hip.linear_dual_supported(rows, e):
                # the two products that read ln_1(x), q/kv and gate/up, as one grid of tiles
                qkv, _ = mvpa_hip.linear_dual(normed.reshape(rows, e), self.attn.qkv_weight(),
                                              self.mlp.gate_up_weight(), out_gated=both[:, e:])
                _, present = self.attn.forward_merged(normed, positional_embedding, channel_embedding, merged,
                                                      attention_mask=attention_mask, use_cache=use_cache,
                                                      qkv=qkv)
            else:
                _, present = self.attn.forward_merged(normed, positional_embedding, channel_embedding, merged,
                                                      attention_mask=attention_mask, use_cache=use_cache)
                self.mlp.activations_into(normed.reshape(rows, e), both[:, e:])
            hidden_states = mvpa_hip.linear(both, self._tail_weight(),
                                            residual=residual.reshape(rows, e)).view(residual.shape)
            next_normed = next_norm(hidden_states) if next_norm is not None else None
            outputs = (hidden_states, present) if use_cache else (hidden_states,)
            return outputs, next_normed
        attn_outputs = self.attn(normed, positional_embedding, channel_embedding,
                                 layer_past=layer_past, attention_mask=attention_mask,
                                 head_mask=head_mask, use_cache=use_cache,
                                 output_attentions=output_attentions)
        attn_output = attn_outputs[0]
        outputs = attn_outputs[1:]
        mlp_output = self.mlp(normed)
        next_normed = None
        if next_norm is not None and residual.dtype == torch.bfloat16:
            hidden_states, next_normed = mvpa_hip.add3_rmsnorm(residual, mlp_output, attn_output,
                                                               next_norm.weight, next_norm.eps)
        else:
            hidden_states = mvpa_hip.add3(residual, mlp_output, attn_output)
            if next_norm is not None:
                next_normed = next_norm(hidden_states)
        if use_cache:
            outputs = (hidden_states,) + outputs
        else:
            outputs = (hidden_states,) + outputs[1:]
        return outputs, next_normed


class MVPFormerModel(nn.Module):
    """models/mvpformer.py:155-402 without the HF base class: h, ln_f, positional_embedding,
    channel_embedding; forward(inputs_embeds=[B,T,C,E]) -> last_hidden_state [B,T,C,E]."""

    def __init__(self, config, gradient_checkpointing=False, flash: bool = True):
        super().__init__()
        self.config = config
        self.embed_dim = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.num_kv_heads = config.n_head_kv
        self.head_dim = self.embed_dim // self.num_heads
        self.embed_kv_dim = self.head_dim * self.num_kv_heads
        self.drop = nn.Dropout(config.embd_pdrop)
        self.h = nn.ModuleList([MVPFormerBlock(config, layer_idx=i, flash=flash)
                                for i in range(config.num_hidden_layers)])
        self.ln_f = RMSNorm(self.embed_dim, eps=config.layer_norm_epsilon)
        self.positional_embedding = nn.Embedding(config.max_position_embeddings, self.embed_dim)
        self.channel_embedding = nn.Embedding(config.max_channel_embeddings, self.embed_dim)
        self.gradient_checkpointing = gradient_checkpointing
        self.apply(self._init_weights)

    def _init_weights(self, module):
        std = self.config.initializer_range                      # models/mvpformer.py:179-188
        if isinstance(module, (nn.Linear, nn.Embedding)):
            module.weight.data.normal_(mean=0.0, std=std)

    def new_cache(self, batch: int, channels: int, max_steps: Optional[int] = None,
                  dtype=torch.bfloat16, device="cuda"):
        """One MvpaKVCache per block for step-by-step decoding (`past_key_values` of forward);
        max_steps defaults to the number of position embeddings."""
        max_steps = self.positional_embedding.num_embeddings if max_steps is None else max_steps
        if max_steps > self.positional_embedding.num_embeddings:
            raise IndexError("more time steps than embedding rows (n_positions)")
        return tuple(MvpaKVCache(batch, self.num_kv_heads, channels, self.head_dim, max_steps,
                                 dtype=dtype, device=device) for _ in self.h)

    def forward(self, input_ids=None, past_key_values=None, inputs_embeds=None, attention_mask=None,
                head_mask=None, use_cache=None, output_attentions=None, position_end=None,
                channel_validity=None, **unused):
        """forward(inputs_embeds=[B,T,C,E]) -> last_hidden_state [B,T,C,E]; with use_cache also the
        per-block `present`s, as the reference returns them in `past_key_values`
        (models/mvpformer.py:290-398).  With past_key_values (one entry per block: the (k, v)
        tuples a use_cache call returned, or the MvpaKVCache objects of new_cache) inputs_embeds
        holds ONE new time step [B,1,C,E] that continues the cached sequence.

        position_end: the T time steps use rows [position_end - T, position_end) of the position
        embedding instead of rows [0, T).  Row j of the T rows in use stands for the distance
        T-1-j between query and key step (layers/mvpa.py:223), so with rows [0, T) the row of a
        given distance moves as a sequence grows; a stream keeps it in place by always ending at
        the same row (MvpaKVCache entries imply position_end = their max_steps).

        channel_validity (extension): [B,C], 1 = channel present; stands for an attention_mask that
        repeats the same 0/1 pattern at every time step, without a look at its values.

        Gradients: with grad mode on and either train() mode or an inputs_embeds that carries a
        graph, the whole-sequence forward is differentiable; in train() mode the embedding,
        residual and attention dropouts of the reference apply there (the attention's as the flash
        layer has it: whole key steps and channels)."""
        if inputs_embeds is None:
            raise NotImplementedError
        grad = torch.is_grad_enabled() and past_key_values is None and (self.training or inputs_embeds.requires_grad)
        if self.training and self.drop.p > 0:
            if not grad:
                raise NotImplementedError("MVPFormer HIP stack: dropout in train() mode goes with the "
                                          "whole-sequence forward in grad mode; call .eval() otherwise")
            inputs_embeds = self.drop(inputs_embeds)                 # models/mvpformer.py:285
        with torch.set_grad_enabled(grad):
            return self._forward(past_key_values, inputs_embeds, attention_mask, use_cache, position_end,
                                 channel_validity)

    def _forward(self, past_key_values, inputs_embeds, attention_mask, use_cache, position_end,
                 channel_validity):
        use_cache = bool(use_cache)      # None = off whatever config.use_cache says: a tensor comes back
        bsz, t_len, c_len, _ = inputs_embeds.shape
        if past_key_values is not None:
            if len(past_key_values) != len(self.h):
                raise ValueError("past_key_values needs one entry per block")
            if t_len != 1:
                raise NotImplementedError("with past_key_values, inputs_embeds holds one new time step")
            first = past_key_values[0]
            past_len = (min(first.length, first.max_steps - 1) if isinstance(first, MvpaKVCache)
                        else first.steps - 1 if isinstance(first, MvpaRingCache)
                        else first[0].shape[2])                  # models/mvpformer.py:241-245
            t_len = past_len + 1
            use_cache = True
            if position_end is None and isinstance(first, MvpaKVCache):
                position_end = first.max_steps
            if position_end is None and isinstance(first, MvpaRingCache):
                position_end = first.steps
        if attention_mask is not None:                           # models/mvpformer.py:262-268
            dt = inputs_embeds.dtype
            attention_mask = attention_mask.view(bsz, -1)[:, None, None, :].to(dtype=dt)
            attention_mask = (1.0 - attention_mask) * torch.finfo(dt).min
            # analysed once for all blocks (one device synchronisation per forward, none per layer)
            attention_mask = KeyMask(attention_mask)
            attention_mask.resolve(bsz, t_len, c_len)
        elif channel_validity is not None:
            # extension: the per-channel validity mask [B,C] (1 = present) handed over as such -
            # what a 0/1 attention_mask that repeats over the time steps amounts to, without the
            # look at its values, so nothing here synchronises with the device
            attention_mask = KeyMask(chan_valid=channel_validity.to(torch.bool))
        # ids are arange(T) / arange(C) (models/mvpformer.py:246-261), so the lookups
        # (models/mvpformer.py:282-283) are leading slices of the embedding tables
        if t_len > self.positional_embedding.num_embeddings or c_len > self.channel_embedding.num_embeddings:
            raise IndexError("more time steps / channels than embedding rows (n_positions / n_channels)")
        pos_lo = 0 if position_end is None else position_end - t_len
        if pos_lo < 0 or pos_lo + t_len > self.positional_embedding.num_embeddings:
            raise IndexError("position_end leaves fewer than T rows of the position embedding")
        position_embeds = self.positional_embedding.weight[pos_lo:pos_lo + t_len][None]
        channel_embeds = self.channel_embedding.weight[:c_len][None]
        hidden_states, normed = inputs_embeds, None
        n_layers = len(self.h)
        presents = () if use_cache else None
        rows = bsz * t_len * c_len
        if (n_layers > 0 and past_key_values is None and not torch.is_grad_enabled() and hidden_states.is_cuda
                and hidden_states.dtype == torch.bfloat16 and self.h[0].norm_fused_supported(rows)):
            # every ln_1 inside the products around it: the statistics of a block's input come out of
            # the previous block's tail product (of one small pass for the first block)
            e = self.embed_dim
            sumsq = mvpa_hip.row_sumsq(hidden_states.reshape(rows, e))
            both = torch.empty((rows, e + self.h[0].mlp.down_proj.in_features), dtype=torch.bfloat16,
                               device=hidden_states.device)
            for block in self.h:
                outputs, sumsq = block.forward_norm_fused(hidden_states, sumsq, position_embeds, channel_embeds,
                                                          attention_mask=attention_mask, use_cache=use_cache,
                                                          both=both)
                hidden_states = outputs[0]
                if use_cache:
                    presents = presents + (outputs[1],)
            out = self.ln_f(hidden_states).view(bsz, inputs_embeds.shape[1], c_len, -1)
            return (out, presents) if use_cache else out
        for i, block in enumerate(self.h):
            next_norm = self.h[i + 1].ln_1 if i + 1 < n_layers else self.ln_f
            layer_past = past_key_values[i] if past_key_values is not None else None
            outputs, normed = block.forward_fused(hidden_states, normed, next_norm, position_embeds,
                                                  channel_embeds, layer_past=layer_past,
                                                  attention_mask=attention_mask, use_cache=use_cache)
            hidden_states = outputs[0]
            if use_cache:
                presents = presents + (outputs[1],)              # models/mvpformer.py:366-367
        if normed is None:                                       # no blocks
            normed = self.ln_f(hidden_states)
        out = normed.view(bsz, inputs_embeds.shape[1], c_len, -1)
        return (out, presents) if use_cache else out


class MVPFormerHead(BrainDecider):
    def __init__(self, size: int, size_out: Optional[int] = None) -> None:
        super().__init__()
        self.head = nn.Linear(size, size_out if size_out is not None else size, bias=False)

    def forward(self, x: torch.Tensor):
        if x.is_cuda and x.dtype == torch.bfloat16:
            if torch.is_grad_enabled() and (x.requires_grad or self.training):
                return AG.linear(x, self.head.weight)
            with torch.no_grad():
                return mvpa_hip.linear(x, self.head.weight.to(torch.bfloat16))
        return self.head(x)


class HMVPFormer(BrainModel):
    """Inference part of the reference's harness: encoder -> stack -> head
    (models/mvpformer.py:405-479, 596-607, 749-764).  Sub-module names match the reference so
    its `base_model` / `head_model` state dicts load key for key."""

    def __init__(self, gpt_config: MVPFormerConfig, encoder: BrainEncoder, head: BrainDecider,
                 flash: bool = True, base_model: str = "", head_model: str = "") -> None:
        super().__init__()
        self.gpt_config = gpt_config
        self.mvpformer = MVPFormerModel(gpt_config, flash=flash)
        self.head = head
        self.encoder = encoder
        self.seizure_embeddings = nn.Parameter(
            torch.normal(mean=0, std=1.0 / encoder.size_input, size=(3, encoder.size_input)))
        self.base_model = base_model
        if base_model != "" or head_model != "":                   # models/mvpformer.py:470-479
            self._load_checkpoint(_load_weights(base_model), _load_weights(head_model))

    def _load_checkpoint(self, base_weights, head_weights):
        """models/mvpformer.py:481-485: the base state dict must match key for key (strict); the
        encoder's norm weight is reset to ones, as there."""
        if base_weights is not None:
            base_weights = dict(base_weights)
            base_weights["encoder.ln.weight"] = torch.ones_like(self.encoder.ln.weight)
            self.load_state_dict(base_weights, strict=True)

    def load_reference_state_dicts(self, base_model_sd=None, head_model_sd=None):
        """Load state dicts saved by the reference's modules (the `base_model` / `head_model` files of
        models/mvpformer.py:470-479, already read with torch.load(..., weights_only=True)), under
        this class's checkpoint policy.  Returns self."""
        self._load_checkpoint(base_model_sd, head_model_sd)
        return self

    def _grad_mode(self):
        """Grad mode of the scoring methods: on only in train() mode under an enabled grad mode."""
        return torch.set_grad_enabled(torch.is_grad_enabled() and self.training)

    def _common_forward(self, batch: torch.Tensor, attention_mask=None):
        """batch [B, n_seg, ch, len] -> (last_hidden_state [B,T,C,E], input_embeds [B,T,C,E])."""
        with self._grad_mode():
            return self._common_forward_impl(batch, attention_mask)

    def _common_forward_impl(self, batch: torch.Tensor, attention_mask=None):
        bsz, seg_n, ch, seg = batch.shape
        out_enc = self.encoder(batch.reshape(bsz * seg_n * ch, seg))
        input_embeds = out_enc.view(bsz, seg_n, ch, -1)
        out = self.mvpformer(inputs_embeds=input_embeds, attention_mask=attention_mask)
        return out, input_embeds

    @torch.no_grad()
    def classify_step(self, segment: torch.Tensor, past=None, max_steps: Optional[int] = None):
        """Classification score of a stream, one segment at a time: segment [B, ch, len] is the
        newest one, `past` what the previous call returned (None at the start of a stream).
        Returns (logits, past).  Each call runs the encoder on the new segment only and one
        decoding step of every block against the cached keys and values.

        What a stream computes: in this model the newest time step keeps the content term for
        EVERY key while older steps only keep it inside the window of 10 (layers/mvpa.py:231-245).
        A decoding step is always the newest step, so from the second block on the cached keys and
        values of a step are the ones it produced as the newest step of its own, shorter, window.
        For streams of at most 12 segments (the window never bites) or a single block this is
        exactly the full forward over the segments so far with its position rows ending at
        max_steps (forward(position_end=max_steps)), and at step max_steps classify() on the whole
        window.  For longer streams with two or more blocks it is a different function of the
        same segments - every step computed with full content attention at the time it arrived -
        and the two differ by far more than rounding (tests/test_model_gpu.py measures it).  After
        max_steps segments the oldest one drops out of the caches at every step."""
        bsz, ch, seg = segment.shape
        embeds = self.encoder(segment.reshape(bsz * ch, seg)).view(bsz, 1, ch, -1)
        if past is None:
            past = self.mvpformer.new_cache(bsz, ch, max_steps, dtype=embeds.dtype, device=embeds.device)
            out, past = self._first_step(embeds, past)
        else:
            out, past = self.mvpformer(inputs_embeds=embeds, past_key_values=past)
        return self.head(out[:, -1].float().mean(dim=1).to(out.dtype)), past

    def capture_stream(self, past, segment_like: torch.Tensor, predict: bool = False):
        """Turn a stream whose window is full into a replayable HIP graph.  `past` is what
        classify_step returned once max_steps segments were in (MvpaKVCache per block);
        segment_like a tensor shaped like one segment batch [B, ch, len].  Returns a callable
        step(segment) -> logits that copies the segment into a fixed buffer and replays the graph
        of one classify_step on ring caches (the caches are copied; `past` is left alone).  The
        returned logits tensor is overwritten by the next call.  predict=True captures predict_step
        instead (`past` as predict_step returned it): step(segment) -> (similarity, prediction),
        the similarity scoring the forecast of the call before."""
        forecast = None
        if predict:
            past, forecast = past
            forecast = forecast.clone()
        clock = MvpaRingClock(past[0].max_steps, past[0].max_steps - 1, segment_like.device)
        rings = tuple(MvpaRingCache.from_cache(c, clock) for c in past)     # one clock for all blocks
        inp = segment_like.clone()

        def one_step():
            clock.advance()
            bsz, ch, seg = inp.shape
            embeds = self.encoder(inp.reshape(bsz * ch, seg)).view(bsz, 1, ch, -1)
            out, _ = self.mvpformer(inputs_embeds=embeds, past_key_values=rings)
            if predict:
                sim = torch.cosine_similarity(embeds[:, 0].float(), forecast.float(), dim=-1)
                forecast.copy_(self.head(out[:, -1]))
                return sim, forecast
            return self.head(out[:, -1].float().mean(dim=1).to(out.dtype))

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        saved = [(r.k.clone(), r.v.clone()) for r in rings]
        head0 = clock.head32.clone()
        forecast0 = forecast.clone() if predict else None
        with torch.cuda.stream(side):
            for _ in range(2):                      # warm-up: fills every host-side cache of the path
                one_step()
        torch.cuda.current_stream().wait_stream(side)
        for r, (k0, v0) in zip(rings, saved):       # the warm-up steps wrote into the rings
            r.k.copy_(k0)
            r.v.copy_(v0)
        clock.head32.copy_(head0)
        if predict:
            forecast.copy_(forecast0)
        del saved
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = one_step()

        def step(segment: torch.Tensor) -> torch.Tensor:
            inp.copy_(segment)
            graph.replay()
            return logits

        step.rings, step.graph = rings, graph
        return step

    def _first_step(self, embeds, caches):
        """The first segment of a stream through the full forward; its keys and values seed the
        caches."""
        out, presents = self.mvpformer(inputs_embeds=embeds, use_cache=True,
                                       position_end=caches[0].max_steps)
        for cache, (k, v) in zip(caches, presents):
            cache.append(k[:, :, 0], v[:, :, 0])
        return out, caches

    def predict_next_segment(self, batch: torch.Tensor):
        """Generative scoring of models/mvpformer.py:749-764: cosine similarity between the head's
        prediction at segment t and the encoding of segment t+1, per channel."""
        with self._grad_mode():
            return self._predict_next_segment(batch)

    def _predict_next_segment(self, batch: torch.Tensor):
        out, enc = self._common_forward(batch)
        out = self.head(out)
        if torch.is_grad_enabled():
            return torch.cosine_similarity(enc[:, 1:].float(), out[:, :-1].float(), dim=-1)
        if enc.is_cuda and enc.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and enc.shape[-1] % 8 == 0:
            return mvpa_hip.cosine_similarity_steps(enc, out)
        return torch.cosine_similarity(enc[:, 1:].float(), out[:, :-1].float(), dim=-1)

    @torch.no_grad()
    def predict_step(self, segment: torch.Tensor, past=None, max_steps: Optional[int] = None):
        """predict_next_segment for a stream, one segment [B, ch, len] at a time.  Returns
        (similarity, prediction, past): `prediction` [B, ch, E] is the head's forecast of the NEXT
        segment's encoding, `similarity` [B, ch] the cosine similarity between this segment's
        encoding and the forecast the previous call made for it (None on the first call) - the
        column of predict_next_segment's result that this segment closes (equal to it for streams
        of at most 12 segments or one block; see classify_step for longer ones).  `past` carries
        the caches and the last forecast from call to call."""
        bsz, ch, seg = segment.shape
        embeds = self.encoder(segment.reshape(bsz * ch, seg)).view(bsz, 1, ch, -1)
        caches, forecast = (None, None) if past is None else past
        if caches is None:
            caches = self.mvpformer.new_cache(bsz, ch, max_steps, dtype=embeds.dtype, device=embeds.device)
            out, caches = self._first_step(embeds, caches)
        else:
            out, caches = self.mvpformer(inputs_embeds=embeds, past_key_values=caches)
        similarity = None
        if forecast is not None:
            similarity = torch.cosine_similarity(embeds[:, 0].float(), forecast.float(), dim=-1)
        prediction = self.head(out[:, -1])
        return similarity, prediction, (caches, prediction)

    def classify(self, batch: torch.Tensor):
        """Classification scoring of models/mvpformer.py:947-953: head(mean over channels of the
        last segment's hidden state)."""
        with self._grad_mode():
            out, _ = self._common_forward(batch)
            return self.head(out[:, -1].float().mean(dim=1).to(out.dtype))


def _load_weights(path: str):
    """torch.load(path, weights_only=True), None for an empty or missing path
    (models/mvpformer.py:471-478)."""
    if path == "":
        return None
    try:
        return torch.load(path, weights_only=True, map_location="cpu")
    except FileNotFoundError:
        return None


class ClassificationHMVPFormer(HMVPFormer):
    """The classification harness's checkpoint policy (models/mvpformer.py:845-904) on the inference
    model: a base state dict whose head has another shape loses that head; with adapters on, only
    adapter, head and encoder.proj_* keys may be missing from it; the head state dict must bring
    the head (and the adapters, with adapters on); `class_loss.weight` is the only key that may be
    unknown."""

    def _load_checkpoint(self, base_weights, head_weights):
        lora = bool(self.gpt_config.lora)
        if base_weights is not None:
            base_weights = dict(base_weights)
            if ("head.head.weight" in base_weights
                    and base_weights["head.head.weight"].shape != self.head.head.weight.shape):
                del base_weights["head.head.weight"]
            miss_key, un_key = self.load_state_dict(base_weights, strict=False)
            if lora:
                miss_key = [k for k in miss_key
                            if "lora" not in k.lower() and "head" not in k.lower()
                            and "encoder.proj_" not in k.lower()]
                if miss_key:
                    raise AttributeError(
                        f"Parameters {miss_key} are missing from the base model and are not trainable.")
            elif miss_key:
                raise AttributeError(f"Parameters {list(miss_key)} are missing from the base model.")
            if len(un_key) > 0:
                raise AttributeError(f"Parameters {list(un_key)} are unknown in the base model.")
        if head_weights is not None:
            miss_key, un_key = self.load_state_dict(dict(head_weights), strict=False)
            needed = [k for k in miss_key
                      if "head" in k.lower() or (lora and "lora" in k.lower())]
            if needed:
                raise AttributeError(f"Parameters {needed} are missing from the head model.")
            if len(un_key) > 0 and list(un_key) != ["class_loss.weight"]:
                raise AttributeError(f"Parameters {list(un_key)} are unknown in the model.")
