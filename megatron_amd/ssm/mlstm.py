"""mLSTM mixer: the outer-product (matrix) memory cell introduced with xLSTM
(Beck et al., "xLSTM: Extended Long Short-Term Memory"): exponential input gate,
log-space gates squashed by cap * tanh(. / cap), and a running-maximum stabiliser.

Per head: S_t = e^{f+m'-m} S + e^{i-m} k v^T, n_t likewise with k,
m = max(f + m', i) (m starts at 0), o = S^T q / (max(|n.q|, e^{-m}) + 1e-6);
o is RMS-normalised per head, scaled by a learned weight, gated by
sigmoid(W_g h) and projected out.  q/k/v/output-gate projections are one fused
GEMM in the compute dtype; the two gate projections (2*heads rows) are a
separate fp32 GEMM because their result feeds log-space recurrences.  State
(S, n, m) is fp32 per request slot (ops.ragged.mlstm_scan)."""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class MLSTMMixer(nn.Module):
    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float,
                 state_name: str, dtype=torch.bfloat16):
        super().__init__()
        self.heads, self.dim, self.vdim = heads, dim, vdim
        self.gate_cap, self.eps = gate_cap, eps
        self.state_name = state_name
        rows = 2 * heads * dim + 2 * heads * vdim
        self.w_in = nn.Parameter(torch.zeros(rows, hidden, dtype=dtype))      # [q; k; v; g]
        self.w_gates = nn.Parameter(torch.zeros(2 * heads, hidden, dtype=torch.float32))  # [i; f]
        self.bias_i = nn.Parameter(torch.zeros(heads, dtype=torch.float32))
        self.bias_f = nn.Parameter(torch.zeros(heads, dtype=torch.float32))
        self.norm_weight = nn.Parameter(torch.ones(heads * vdim, dtype=torch.float32))
        self.w_out = nn.Parameter(torch.zeros(hidden, heads * vdim, dtype=dtype))

    def cache_spec(self):
        return {}

    def state_spec(self):
        n = self.state_name
        return {n + ".S": ((self.heads, self.dim, self.vdim), torch.float32),
                n + ".n": ((self.heads, self.dim), torch.float32),
                n + ".m": ((self.heads,), torch.float32)}

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        qkvg = F.linear(h, self.w_in)
        gates = F.linear(h.float(), self.w_gates)
        n = self.state_name
        o = R.mlstm_scan(qkvg, gates, self.bias_i, self.bias_f, self.norm_weight,
                         self.heads, self.dim, self.vdim, self.gate_cap, self.eps,
                         ctx.states[n + ".S"], ctx.states[n + ".n"], ctx.states[n + ".m"],
                         ctx.batch, h.dtype)
        return F.linear(o, self.w_out)
