"""Hyper-connections: several residual streams in place of one.

A sublayer reads the blend u = sum_s read[s] x_s and computes y = f(norm(u)); the
new streams are x'_t = sum_s mix[s, t] x_s + write[t] y, every x'_t formed from the
streams as they were before the sublayer (mix[s, t] weighs old stream s in new
stream t).  With one stream and read = write = mix = 1 this
is the ordinary pre-norm residual, which is how single-stream models use the
same fused kernel (ops.ragged.hc_mix_norm: stream update of the previous
sublayer + read + RMS norm of the next in one pass over the streams).
"""

from __future__ import annotations

import torch
import torch.nn as nn


class HyperConnection(nn.Module):
    """Read / write / mix weights of one sublayer (fp32)."""

    def __init__(self, streams: int):
        super().__init__()
        self.streams = streams
        self.read = nn.Parameter(torch.ones(streams, dtype=torch.float32))
        self.write = nn.Parameter(torch.ones(streams, dtype=torch.float32))
        self.mix = nn.Parameter(torch.eye(streams, dtype=torch.float32))
