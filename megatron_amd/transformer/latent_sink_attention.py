"""Latent attention with a softmax sink, an output gate and a shareable cache.

Keys and values are up-projections of one low-rank latent per token plus one
rotated key part shared by all heads (multi-head latent attention, DeepSeek-V2);
only [normed latent | rotated key part] is cached, in a paged pool.  This module
always runs the absorbed form: the key up-projection is folded into the query
(q~_h = W_uk,h^T q_h) so scores are taken against the cached rows directly, and
the value up-projection is applied to the probability-weighted latent sum.

Extras over megatron_amd.transformer.multi_latent_attention:
  * ragged batches (prompt portions beside single decoded tokens) over the
    paged pool of a HybridInferenceContext,
  * a per-head sink logit in the softmax denominator (no key, no value),
  * a per-head sigmoid output gate read from the layer input,
  * ``kv_source``: a layer may own no down-projection and read another
    layer's pool,
  * RoPE (rotate-half) with optional YaRN scaling on the rotated part; the
    score scale is a given constant.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class LatentSinkAttention(nn.Module):
    def __init__(self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 q_rank: int, scale: float, rot_dims: int, rot_base: float, rot_scaling: Optional[dict],
                 eps: float, max_positions: int, cache_name: str, owns_cache: bool,
                 dtype=torch.bfloat16):
        super().__init__()
        self.heads, self.dim, self.rot_dim, self.vdim = heads, dim, rot_dim, vdim
        self.kv_rank, self.q_rank, self.scale, self.eps = kv_rank, q_rank, scale, eps
        self.rot_dims = rot_dims
        self.cache_name, self.owns_cache = cache_name, owns_cache
        rows = q_rank + (kv_rank + rot_dim if owns_cache else 0) + heads
        self.w_in = nn.Parameter(torch.zeros(rows, hidden, dtype=dtype))  # [q down; (kv down); gate]
        self.q_norm = nn.Parameter(torch.ones(q_rank, dtype=torch.float32))
        if owns_cache:
            self.kv_norm = nn.Parameter(torch.ones(kv_rank, dtype=torch.float32))
        self.w_uq = nn.Parameter(torch.zeros(heads * (dim + rot_dim), q_rank, dtype=dtype))
        self.w_uk = nn.Parameter(torch.zeros(heads, dim, kv_rank, dtype=dtype))
        self.w_uv = nn.Parameter(torch.zeros(heads, vdim, kv_rank, dtype=dtype))
        self.sink = nn.Parameter(torch.zeros(heads, dtype=torch.float32))
        self.w_out = nn.Parameter(torch.zeros(hidden, heads * vdim, dtype=dtype))
        cos, sin = R.rope_table(max_positions, rot_dims, rot_base, rot_scaling)
        self.register_buffer("cos", cos, persistent=False)
        self.register_buffer("sin", sin, persistent=False)

    def cache_spec(self):
        return {self.cache_name: self.kv_rank + self.rot_dim} if self.owns_cache else {}

    def state_spec(self):
        return {}

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        batch = ctx.batch
        T = h.shape[0]
        H, D, rd, r = self.heads, self.dim, self.rot_dim, self.kv_rank
        a = F.linear(h, self.w_in)
        pool = ctx.pools[self.cache_name]
        if self.owns_cache:
            R.latent_kv_store(a[:, self.q_rank : self.q_rank + r + rd], self.kv_norm, self.eps,
                              self.cos, self.sin, self.rot_dims, r, pool, batch)
        cq = R.latent_q_prepare(a[:, : self.q_rank], self.q_norm, self.eps, h.dtype)
        q = F.linear(cq, self.w_uq).view(T, H, D + rd)
        q_abs = torch.bmm(q[..., :D].transpose(0, 1), self.w_uk).transpose(0, 1)  # [T, H, r]
        lat_q = R.assemble_latent_q(q_abs, q[..., D:], self.cos, self.sin, self.rot_dims, batch)
        c_hat = R.latent_sink_attention(lat_q, pool, r, self.sink, self.scale, batch)  # [T, H, r]
        o = torch.bmm(c_hat.transpose(0, 1), self.w_uv.transpose(1, 2)).transpose(0, 1)  # [T, H, vd] view
        o = R.gate_heads(o, a[:, a.shape[1] - H :], H)                                   # [T, H * vd]
        return F.linear(o, self.w_out)
