"""Residual causal depthwise convolution over time in front of a mixer
("canon" layer): h <- h + conv(h), conv(h)_t = sum_j w[:, j] h_{t-taps+1+j}, with the
sequence zero-padded on the left.  The last taps-1 inputs are per-sequence state
so a sequence can be fed in portions of any size."""

from __future__ import annotations

import torch
import torch.nn as nn

from megatron_amd.ops import ragged as R


class CanonConv(nn.Module):
    def __init__(self, width: int, taps: int, state_name: str):
        super().__init__()
        self.taps = taps
        self.state_name = state_name
        self.weight = nn.Parameter(torch.zeros(width, taps, dtype=torch.float32))

    def state_spec(self):
        return {self.state_name: ((self.taps - 1, self.weight.shape[0]), torch.float32)}

    def forward(self, h: torch.Tensor, ctx, out_dtype) -> torch.Tensor:
        return R.canon_conv(h, self.weight, ctx.states[self.state_name], ctx.batch, out_dtype)
