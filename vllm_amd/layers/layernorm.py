"""RMSNorm / LayerNorm wrappers dispatching to custom ops
(reference: vllm/model_executor/layers/layernorm.py)."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from vllm_amd import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6, dtype=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype),
                                   requires_grad=False)
        self.eps = eps

    def forward(
        self, x: torch.Tensor, residual: Optional[torch.Tensor] = None
    ):
        if residual is None:
            return ops.rms_norm(x, self.weight, self.eps)
        return ops.fused_add_rms_norm(x, residual, self.weight, self.eps)

    def cast(self, x: torch.Tensor, out_dtype) -> torch.Tensor:
        """Norm computed in fp32 from x of any dtype, stored as
        out_dtype (an fp32 residual stream feeding a 16-bit GEMM)."""
        return ops.rms_norm_cast(x, self.weight, self.eps, out_dtype)

    def add_into(self, residual: torch.Tensor, y: torch.Tensor,
                 out_dtype=None) -> torch.Tensor:
        """Norm on a sublayer's OUTPUT: residual (fp32, in place) +=
        norm(y) * weight in one pass; hands back the updated residual,
        as a copy in out_dtype when the next GEMM wants 16 bits."""
        return ops.add_rms_norm(residual, y, self.weight, self.eps,
                                out_dtype)


class LayerNorm(nn.Module):
    """Plain LayerNorm (OPT family). Uses torch's — not a hot op for the
    benchmark models; HIP fusion comes with the OPT fast path if needed."""

    def __init__(self, hidden_size: int, eps: float = 1e-5, dtype=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype),
                                   requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=dtype),
                                 requires_grad=False)
        self.eps = eps

    def forward(self, x, residual: Optional[torch.Tensor] = None):
        if residual is not None:
            x = x + residual
            residual = x
        out = torch.nn.functional.layer_norm(
            x.float(), (x.shape[-1],), self.weight.float(),
            self.bias.float(), self.eps,
        ).to(x.dtype)
        if residual is not None:
            return out, residual
        return out


class ScalarRMSNorm(nn.Module):
    """RMS norm whose gain is ONE number for all coordinates:
    x / sqrt(mean(x^2) + eps) * g. Always computed in fp32.

    forward(x) returns the normed rows (fp32, or out_dtype);
    add_into(residual, y, mult) does residual += mult * norm(y) in place
    on an fp32 residual stream and can hand back a copy of the updated
    residual in the compute dtype for the next GEMM (one fused pass)."""

    def __init__(self, eps: float = 1e-6):
        super().__init__()
        self.gain = nn.Parameter(torch.ones((), dtype=torch.float32),
                                 requires_grad=False)
        self.eps = eps

    def forward(self, x: torch.Tensor, out_dtype=None) -> torch.Tensor:
        return ops.scalar_rms_norm(x, self.gain, self.eps, out_dtype)

    def add_into(self, residual: torch.Tensor, y: torch.Tensor,
                 mult: float, out_dtype=None) -> torch.Tensor:
        return ops.add_scaled_scalar_norm(residual, y, self.gain,
                                          self.eps, mult, out_dtype)
