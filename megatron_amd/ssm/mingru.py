"""minGRU mixer: an elementwise linear recurrence whose update gate and candidate
are functions of the present input alone (no hidden-state feedback into the
gates), S_t = (1 - z_t) S_{t-1} + z_t c_t with z = sigmoid(W_z h + b_z) and
c = g(W_x h + b_x), g(u) = u + 1/2 for u >= 0 and sigmoid(u) below
(Feng et al., "Were RNNs All We Needed?").  Output W_o (S_t * silu(W_g h)).

The three input projections are one fused GEMM; the recurrence, both gate
non-linearities and the output gate run in one kernel with the state held in
32-bit per request slot (ops.ragged.mingru_scan)."""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class MinGRUMixer(nn.Module):
    def __init__(self, hidden: int, width: int, state_name: str, dtype=torch.bfloat16):
        super().__init__()
        self.width = width
        self.state_name = state_name
        self.w_in = nn.Parameter(torch.zeros(3 * width, hidden, dtype=dtype))  # [z; x; g]
        self.bias_z = nn.Parameter(torch.zeros(width, dtype=torch.float32))
        self.bias_x = nn.Parameter(torch.zeros(width, dtype=torch.float32))
        self.w_out = nn.Parameter(torch.zeros(hidden, width, dtype=dtype))

    def cache_spec(self):
        return {}

    def state_spec(self):
        return {self.state_name: ((self.width,), torch.float32)}

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        zxg = F.linear(h, self.w_in)
        s = R.mingru_scan(zxg, self.bias_z, self.bias_x, ctx.states[self.state_name], ctx.batch, h.dtype)
        return F.linear(s, self.w_out)
