"""Token shift: a mixer reads a per-channel blend of the current and
the previous token's input,

    h~[t] = h[t] + (h[t-1] - h[t]) * mu,

with h[-1] = 0 at the start of a sequence. The previous token of a
chunk's first token comes from per-request state owned by the model
runner (one fp32 row per running request and layer, cleared when a row
is handed to a new request) and the chunk's last input is stored back,
so chunked prefill and decode see exactly the sequence-level recurrence.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from vllm_amd import ops
from vllm_amd.worker.forward_context import get_forward_context


class TokenShift(nn.Module):

    def __init__(self, width: int):
        super().__init__()
        self.mu = nn.Parameter(torch.zeros(width, dtype=torch.float32),
                               requires_grad=False)

    def forward(self, x: torch.Tensor, state_idx: int,
                out_dtype: torch.dtype) -> torch.Tensor:
        """x: [T, width] fp32 rows of the flat batch; state_idx selects
        this layer's slice of the runner's carry tensor."""
        ctx = get_forward_context()
        meta = ctx.attn_metadata
        state = None
        if ctx.shift_states is not None:
            state = ctx.shift_states[state_idx]
        return ops.token_shift(x, self.mu, state, meta.state_rows,
                               meta.query_start_loc, out_dtype)
