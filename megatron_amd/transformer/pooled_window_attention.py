"""Grouped-query attention over a sliding window plus mean-pooled blocks.

Position i attends to the last ``window`` tokens (itself included) and, beside
them, to ONE key/value per block of ``pool`` consecutive tokens that lies
wholly before the window: block b covers positions b*pool .. b*pool+pool-1 and
is visible once b*pool + pool - 1 <= i - window.  A block's key / value is the
mean of its tokens' cached keys / values.  Tokens that left the window while
their block is still incomplete for i are not visible.  Window tokens and
blocks share one softmax.  Cost per query is window + i / pool instead of i.

Other properties, each a constructor parameter:
  * query and key RMS norm taken over the WHOLE projection (all heads at
    once, before the split into heads) with plain weights,
  * ``values_are_keys``: no value projection, the values are the key
    projection before its norm (head g's value = slice g of the raw keys),
  * no positional rotation; the score scale is a given constant.

Cache: two paged pools of a HybridInferenceContext that share the request's
block table: ``<name>`` rows [normed keys | values] per token and
``<name>.pooled`` rows of the same width per completed block
(ceil(page / pool) rows a page).  The step's own rows and the blocks it
completes are written before attention, so whole prompts, portions and decoded
tokens are one path.

The module can own its projections (standalone layer) or run on column slices
of a projection fused with a neighbour (transformer/parallel_mixer.py).
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class PooledWindowAttention(nn.Module):
    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int, pool: int, eps: float, values_are_keys: bool = True,
                 own_projections: bool = True, dtype=torch.bfloat16):
        super().__init__()
        assert heads % kv_heads == 0, "query heads are a multiple of key/value heads"
        assert window >= 1 and pool >= 1
        if values_are_keys:
            assert kv_heads * vdim == kv_heads * dim, "values taken from the key projection have its width"
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.window, self.pool, self.eps = float(scale), int(window), int(pool), float(eps)
        self.values_are_keys = values_are_keys
        self.q_width, self.k_width, self.v_width = heads * dim, kv_heads * dim, kv_heads * vdim
        self.in_rows = self.q_width + self.k_width + (0 if values_are_keys else self.v_width)
        self.out_cols = heads * vdim
        self.q_norm = nn.Parameter(torch.ones(self.q_width, dtype=torch.float32))
        self.k_norm = nn.Parameter(torch.ones(self.k_width, dtype=torch.float32))
        if own_projections:
            self.w_in = nn.Parameter(torch.zeros(self.in_rows, hidden, dtype=dtype))   # [q; k; (v)]
            self.w_out = nn.Parameter(torch.zeros(hidden, self.out_cols, dtype=dtype))

    def pooled_per_page(self, page: int) -> int:
        return (page + self.pool - 1) // self.pool

    def cache_spec(self, name: str, page: int):
        width = self.k_width + self.v_width
        return {name: width, name + ".pooled": (width, self.pooled_per_page(page))}

    def state_spec(self, name: str):
        return {}

    def run(self, proj: torch.Tensor, col0: int, ctx, name: str, out: torch.Tensor, out_col: int,
            out_scale: float = 1.0) -> None:
        """proj[:, col0 : col0 + in_rows] = [q | k | (v)] of the step's tokens;
        writes out[:, out_col : out_col + out_cols] = out_scale * attention."""
        batch = ctx.batch
        pool, pooled = ctx.pools[name], ctx.pools[name + ".pooled"]
        k_off = col0 + self.q_width
        v_off = k_off if self.values_are_keys else k_off + self.k_width
        q = R.qk_norm_store(proj, col0, self.q_width, k_off, self.k_width, v_off, self.v_width,
                            self.q_norm, self.k_norm, self.eps, pool, batch)
        per_page = self.pooled_per_page(batch.block_size)
        R.pool_blocks(pool, pooled, self.pool, per_page, batch)
        R.pooled_window_attention(q, pool, pooled, self.heads, self.kv_heads, self.dim, self.vdim, self.scale,
                                  self.window, self.pool, per_page, batch, out, out_col, out_scale)

    def forward(self, h: torch.Tensor, ctx, name: str) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        out = torch.empty(h.shape[0], self.out_cols, dtype=h.dtype, device=h.device)
        self.run(proj, 0, ctx, name, out, 0)
        return F.linear(out, self.w_out)
