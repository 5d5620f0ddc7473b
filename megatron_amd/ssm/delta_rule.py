"""Generalized delta-rule mixer: a matrix memory per head with a per-channel
decay and a per-channel removal rate along the unit key.

With r, k, v = W_r h, W_k h, W_v h (heads x dim each), per head:
    decay    w = exp(-e^{-1/2} sigmoid(W_w2 tanh(W_w1 h) + w0))    in (e^{-0.607}, 1)
    removal  a = sigmoid(W_a h + b_a)
    unit key u = k / sqrt(sum k^2 + 1e-6)
    S_t = diag(w) S_{t-1} - (a * u)(u^T S_{t-1}) + k v^T          (both terms read S_{t-1})
    o_t = S_t^T r
Each head's o is divided by its root mean square, scaled by a learned weight,
gated by sigmoid(W_g h) and projected out.  (The update family of RWKV-7;
with a = 0 it is a decayed linear-attention memory, with w = 1 and a = 1 the
classic delta rule along u.)

r, k, v, the gate, the removal pre-activation and the decay bottleneck are one
fused GEMM in the compute dtype; everything that enters the recurrence after
the projections (tanh, the second decay matrix, sigmoids, exponentials, the
unit norm) and the state are 32-bit (ops.ragged.delta_rule_scan).  State:
``<name>.S`` [heads, dim, dim] fp32 per request slot.

The module can own its projections (standalone layer) or run on column slices
of a projection fused with a neighbour (transformer/parallel_mixer.py).
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class DeltaRuleMixer(nn.Module):
    def __init__(self, hidden: int, heads: int, dim: int, decay_rank: int, eps: float,
                 own_projections: bool = True, dtype=torch.bfloat16):
        super().__init__()
        self.heads, self.dim, self.decay_rank, self.eps = heads, dim, decay_rank, float(eps)
        hd = heads * dim
        self.width = hd
        self.in_rows = 5 * hd + decay_rank            # [r; k; v; g; a; w1]
        self.out_cols = hd
        self.w2 = nn.Parameter(torch.zeros(hd, decay_rank, dtype=torch.float32))
        self.w0 = nn.Parameter(torch.zeros(hd, dtype=torch.float32))
        self.a_bias = nn.Parameter(torch.zeros(hd, dtype=torch.float32))
        self.norm_weight = nn.Parameter(torch.ones(hd, dtype=torch.float32))
        if own_projections:
            self.w_in = nn.Parameter(torch.zeros(self.in_rows, hidden, dtype=dtype))
            self.w_out = nn.Parameter(torch.zeros(hidden, hd, dtype=dtype))

    def cache_spec(self, name: str, page: int):
        return {}

    def state_spec(self, name: str):
        return {name + ".S": ((self.heads, self.dim, self.dim), torch.float32)}

    def run(self, proj: torch.Tensor, col0: int, ctx, name: str, out: torch.Tensor, out_col: int,
            out_scale: float = 1.0) -> None:
        hd = self.width
        R.delta_rule_scan(proj, col0, col0 + hd, col0 + 2 * hd, col0 + 3 * hd, col0 + 4 * hd, col0 + 5 * hd,
                          self.decay_rank, self.w2, self.w0, self.a_bias, self.norm_weight, self.heads,
                          self.dim, self.eps, ctx.states[name + ".S"], ctx.batch, out, out_col, out_scale)

    def forward(self, h: torch.Tensor, ctx, name: str) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        out = torch.empty(h.shape[0], self.out_cols, dtype=h.dtype, device=h.device)
        self.run(proj, 0, ctx, name, out, 0)
        return F.linear(out, self.w_out)
