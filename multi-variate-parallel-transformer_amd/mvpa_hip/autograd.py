"""Differentiable wrappers of the library's dense ops, for gradients through the layer and stack
modules (the reference trains through layers/mvpa.py:280-337 and models/mvpformer.py:132-147).

Forward passes are the library's kernels.  The backward passes of the bf16 products are the two
plain products dX = dY W and dW = dY^T X on the vendor library through torch.matmul: it reads
the transposed operand in place and splits the long contraction of a weight gradient (a small
[N,K] output over all rows), which this library's GEMM would run on a few dozen tiles.  The
norm's backward is a few fp32 tensor ops.  The attention operator itself is
`attentions.attn.FlashMVPA` (mvpa_backward kernels).
"""
from __future__ import annotations

import torch

import mvpa_hip


def wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class _LinearFn(torch.autograd.Function):
    """y = x @ w^T, bf16, any leading shape of x: forward on the GPU library, backward on the vendor GEMM."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return mvpa_hip.linear(x, w)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        k = x.shape[-1]
        dy2 = dy.reshape(-1, dy.shape[-1]).contiguous()
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = torch.matmul(dy2, w).view(x.shape)                               # [M,N] @ [N,K]
        if ctx.needs_input_grad[1]:
            dw = torch.matmul(dy2.t(), x.reshape(-1, k))                          # [N,M] @ [M,K]
        return dx, dw


class _LinearF32Fn(torch.autograd.Function):
    """The same in fp32 (the library's fp32 MFMA product, forward and both backward products)."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return mvpa_hip.linear_f32(x, w)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1]).contiguous()
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = mvpa_hip.linear_f32(dy2, w.t().contiguous()).view(x.shape)
        if ctx.needs_input_grad[1]:
            dw = mvpa_hip.linear_f32(dy2.t().contiguous(), x.reshape(-1, x.shape[-1]).t().contiguous())
        return dx, dw


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w^T on the GPU library, bf16 or fp32 (differentiably when a gradient is wanted);
    tensors that are not on the GPU take torch's own linear."""
    if x.is_cuda and x.dtype == torch.bfloat16:
        w = w.to(torch.bfloat16)
        if wants_grad(x, w):
            return _LinearFn.apply(x, w)
        return mvpa_hip.linear(x, w.detach())
    if x.is_cuda and x.dtype == torch.float32:
        w = w.to(torch.float32)
        if wants_grad(x, w):
            return _LinearF32Fn.apply(x, w)
        return mvpa_hip.linear_f32(x, w.detach())
    return torch.nn.functional.linear(x, w.to(x.dtype))


class _RMSNormFn(torch.autograd.Function):
    """y = x * rsqrt(mean(x^2) + eps) * w; forward on the library's kernel, backward in fp32."""

    @staticmethod
    def forward(ctx, x, w, eps, out_dtype):
        ctx.save_for_backward(x, w)
        ctx.eps = eps
        return mvpa_hip.rmsnorm(x, w, eps, out_dtype=out_dtype)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        xf, wf, g = x.float(), w.float(), dy.float()
        r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + ctx.eps)
        gw = g * wf
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = (r * gw - xf * r.pow(3) * (xf * gw).mean(-1, keepdim=True)).to(x.dtype)
        if ctx.needs_input_grad[1]:
            dw = (g * xf * r).reshape(-1, x.shape[-1]).sum(0).to(w.dtype)
        return dx, dw, None, None


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype=None) -> torch.Tensor:
    if wants_grad(x, w):
        return _RMSNormFn.apply(x, w, eps, out_dtype)
    return mvpa_hip.rmsnorm(x, w, eps, out_dtype=out_dtype)
