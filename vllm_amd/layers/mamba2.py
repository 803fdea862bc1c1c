"""State-space-duality (Mamba-2) mixer.

One input projection yields [z | x | B | C | dt] (widths inner, inner,
G*N, G*N, heads with inner = heads * head_dim). x, B and C pass one
per-channel causal convolution with bias and silu; per head h (using
B/C group h // (heads/G)) the recurrence runs in fp32:

    dt' = softplus(dt + dt_bias)                (no clamp)
    S   = exp(-exp(A_log) dt') S + dt' x B^T    (S is [head_dim, N])
    y   = S C + D x

y is multiplied by silu(z), RMS-normed in `norm_groups` equal parts
(gate BEFORE the norm), scaled by a weight and projected out.

Per-request state lives in runner rows: the convolution's last taps-1
inputs (compute dtype) and S (fp32). Rows are cleared when handed to a
request, so chunked prefill and decode follow the sequence-level
recurrence exactly.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from vllm_amd import ops
from vllm_amd.layers.linear import ReplicatedLinear
from vllm_amd.worker.forward_context import get_forward_context


class Mamba2Mixer(nn.Module):

    def __init__(self, width: int, heads: int, head_dim: int, state: int,
                 groups: int, conv_taps: int, norm_groups: int, eps: float,
                 state_idx: int, dtype: torch.dtype):
        super().__init__()
        assert heads % groups == 0
        self.heads, self.head_dim = heads, head_dim
        self.state, self.groups = state, groups
        self.taps, self.norm_groups = conv_taps, norm_groups
        self.eps = eps
        self.state_idx = state_idx
        self.inner = heads * head_dim
        assert self.inner % norm_groups == 0
        self.conv_dim = self.inner + 2 * groups * state
        self.in_proj = ReplicatedLinear(
            width, 2 * self.inner + 2 * groups * state + heads,
            bias=False, dtype=dtype)
        self.conv_weight = nn.Parameter(
            torch.zeros(self.conv_dim, conv_taps, dtype=dtype),
            requires_grad=False)
        self.conv_bias = nn.Parameter(
            torch.zeros(self.conv_dim, dtype=dtype), requires_grad=False)
        f32 = torch.float32
        self.dt_bias = nn.Parameter(torch.zeros(heads, dtype=f32),
                                    requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(heads, dtype=f32),
                                  requires_grad=False)
        self.D = nn.Parameter(torch.ones(heads, dtype=f32),
                              requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(self.inner, dtype=f32),
                                        requires_grad=False)
        self.out_proj = ReplicatedLinear(self.inner, width, bias=False,
                                         dtype=dtype)

    @staticmethod
    def state_shapes(mx: dict) -> tuple[tuple, tuple]:
        """(conv tail, recurrent state) shapes per request row."""
        inner = mx["heads"] * mx["vdim"]
        return ((inner + 2 * mx["groups"] * mx["state"],
                 max(int(mx["conv"]) - 1, 0)),
                (mx["heads"], mx["vdim"], mx["state"]))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_forward_context()
        meta = ctx.attn_metadata
        conv_state = ssm_state = None
        if ctx.layer_states is not None:
            conv_state, ssm_state = ctx.layer_states[self.state_idx]
        T = h.shape[0]
        p = self.in_proj(h)
        a, b = self.inner, self.inner + self.conv_dim
        z, xbc, dt = p[:, :a], p[:, a:b], p[:, b:]
        # The conv output only feeds the recurrence, which is fp32.
        xbc = ops.causal_conv_silu(
            xbc, self.conv_weight, self.conv_bias, conv_state,
            meta.state_rows, meta.query_start_loc,
            out_dtype=torch.float32)
        y = ops.ssd_scan(xbc, self.heads, self.head_dim, self.groups,
                         self.state, dt, self.dt_bias, self.A_log, self.D,
                         ssm_state, meta.state_rows, meta.query_start_loc,
                         max_query_len=meta.max_query_len)
        y = ops.gated_group_rms_norm(
            y.view(T, self.inner), z, self.norm_weight, self.eps,
            self.norm_groups, h.dtype)
        return self.out_proj(y)
