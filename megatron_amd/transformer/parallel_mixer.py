"""Two sequence mixers side by side on the same input:
y = left_scale * left(h) + right_scale * right(h).

Both input projections run as ONE GEMM ([left rows; right rows] x h) and both
output projections as ONE GEMM over the concatenated mixer outputs
([left_scale * o_left | right_scale * o_right] x [W_o,left | W_o,right]^T): each
mixer reads its column slice of the fused projection and writes its scaled
result into its column slice of the shared output buffer, so the weighted sum
is formed inside the output GEMM's accumulation and costs nothing.

The halves are any modules with ``in_rows``, ``out_cols``,
``run(proj, col0, ctx, name, out, out_col, out_scale)``, ``cache_spec`` and
``state_spec`` (transformer/pooled_window_attention.py, ssm/delta_rule.py).
Caches and states are named at call time (``<name>.left``, ``<name>.right``):
layers that share weights keep caches and states of their own.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


class ParallelMixer(nn.Module):
    def __init__(self, hidden: int, left: nn.Module, right: nn.Module, left_scale: float, right_scale: float,
                 dtype=torch.bfloat16):
        super().__init__()
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.w_in = nn.Parameter(torch.zeros(left.in_rows + right.in_rows, hidden, dtype=dtype))
        self.w_out = nn.Parameter(torch.zeros(hidden, left.out_cols + right.out_cols, dtype=dtype))

    def cache_spec(self, name: str, page: int):
        return {**self.left.cache_spec(name + ".left", page), **self.right.cache_spec(name + ".right", page)}

    def state_spec(self, name: str):
        return {**self.left.state_spec(name + ".left"), **self.right.state_spec(name + ".right")}

    def forward(self, h: torch.Tensor, ctx, name: str) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        out = torch.empty(h.shape[0], self.w_out.shape[1], dtype=h.dtype, device=h.device)
        self.left.run(proj, 0, ctx, name + ".left", out, 0, self.left_scale)
        self.right.run(proj, self.left.in_rows, ctx, name + ".right", out, self.left.out_cols, self.right_scale)
        return F.linear(out, self.w_out)
