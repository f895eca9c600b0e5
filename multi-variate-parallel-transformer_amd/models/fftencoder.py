"""Wavelet segment encoder (the reference's WaveEncoder, models/fftencoder.py:49-106):
multilevel db4 analysis with periodic extension -> RMSNorm(eps 1e-5) -> bias-free projection.
All three stages run through the HIP library; there is no dependency on a wavelet package.
"""
from __future__ import annotations

import torch
from torch import Tensor, nn

import mvpa_hip
from mvpa_hip import autograd as AG
from models import BrainEncoder


class RMSNorm(nn.Module):
    """weight-only RMSNorm with the parameter name the reference's norm uses."""

    def __init__(self, size: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(size))

    def forward(self, x: Tensor) -> Tensor:
        if torch.is_grad_enabled() and (x.requires_grad or self.training):
            return AG.rmsnorm(x, self.weight, self.eps)
        return mvpa_hip.rmsnorm(x, self.weight, self.eps)


class WaveEncoder(BrainEncoder):
    def __init__(self, size_input: int, size_output: int, wavelet: str = "db4",
                 gradient_checkpointing: bool = False) -> None:
        super().__init__()
        if wavelet != "db4":
            raise NotImplementedError("only the db4 wavelet of the shipped configurations is implemented")
        self.size_input = size_input
        self.size_output = size_output
        self.gradient_checkpointing = gradient_checkpointing
        self.levels, self.sizes = mvpa_hip.dwt_sizes(size_input)      # models/fftencoder.py:70-78
        self.dwt_size = sum(self.sizes)
        self.ln = RMSNorm(self.dwt_size, eps=1e-5)
        self.proj = nn.Linear(self.dwt_size, size_output, bias=False)
        self._proj_padded = None
        self._proj_key = None

    @torch.no_grad()
    def block(self, x: Tensor) -> Tensor:
        """[M, L] -> [M, dwt_size] float32 coefficients [cA_L, cD_L, ..., cD_1]."""
        return mvpa_hip.wavedec_db4(x.float())

    def _padded_k(self) -> int:
        """dwt_size (550 for 512-sample segments) rounded up to whole 64-element k-blocks: the
        GEMM then fetches whole cache lines and needs no tail block."""
        return (self.dwt_size + 63) // 64 * 64

    def _padded_weight(self) -> Tensor:
        """bf16 copy of proj.weight with its rows zero-padded to _padded_k() elements."""
        w = self.proj.weight
        key = (w.data_ptr(), w._version)
        if self._proj_key != key:
            kp = self._padded_k()
            buf = torch.zeros((w.shape[0], kp), dtype=torch.bfloat16, device=w.device)
            buf[:, : self.dwt_size] = w.detach().to(torch.bfloat16)
            self._proj_padded, self._proj_key = buf, key
        return self._proj_padded

    def forward(self, x: Tensor) -> Tensor:
        """x [M, L] -> [M, size_output]; bf16 output (the model's compute dtype).  In train() mode
        under grad the norm and the projection are differentiable; the wavelet transform has no
        parameters and carries no gradient (models/fftencoder.py:80: no_grad)."""
        if torch.is_grad_enabled() and self.training:
            return self._forward_autograd(x)
        with torch.no_grad():
            return self._forward_fused(x)

    def _forward_autograd(self, x: Tensor) -> Tensor:
        pad = self._padded_k() - self.dwt_size
        coeffs = self.block(x)                                                  # fp32, no gradient
        normed = AG.rmsnorm(coeffs, self.ln.weight, 1e-5, out_dtype=torch.bfloat16)
        # whole 64-element k-blocks, as on the inference path: the zero columns contribute nothing
        return AG.linear(torch.nn.functional.pad(normed, (0, pad)),
                         torch.nn.functional.pad(self.proj.weight.to(torch.bfloat16), (0, pad)))

    def _forward_fused(self, x: Tensor) -> Tensor:
        m = x.shape[0]
        kp = self._padded_k()
        coeffs = mvpa_hip.wavedec_db4(x.float(), pitch=kp, zero_pad=False)   # [M, dwt] view, pitch kp
        normed = torch.empty((m, kp), dtype=torch.bfloat16, device=x.device)
        normed[:, self.dwt_size:].zero_()
        mvpa_hip.rmsnorm(coeffs, self.ln.weight, 1e-5, out=normed[:, : self.dwt_size])
        w = self._padded_weight()
        return mvpa_hip.linear(normed, w)          # the zero padding contributes nothing

    def encode(self, x: Tensor) -> Tensor:
        return self.forward(x)
