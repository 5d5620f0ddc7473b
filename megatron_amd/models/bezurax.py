"""Bezurax: a decoder-only LM whose layers run two sequence mixers side by
side on the same normed input (grouped-query attention over a sliding window
plus mean-pooled blocks, and a generalized delta-rule memory) in parallel with
a routed-experts feed-forward:

    x <- x + (mixer(norm1(x)) + ff(norm2(x)))

with RMS norms taken in groups of the width, a plain fp32 residual stream, a
tied embedding / output matrix with a logit scale, and layers that may reuse
another layer's weights (with a cache and state of their own).

The model only has a ragged forward (see models/bezutar.py): a flat batch of
tokens laid out by the engine's cache/state manager.  Everything is read from
config.json: sizes, layer order, weight sharing and every constant.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.models.bezutar import InferenceSpec
from megatron_amd.moe.routed_experts import RoutedExpertsMLP
from megatron_amd.ops import ragged as R
from megatron_amd.ssm.delta_rule import DeltaRuleMixer
from megatron_amd.transformer.parallel_mixer import ParallelMixer
from megatron_amd.transformer.pooled_window_attention import PooledWindowAttention


@dataclass
class BezuraxConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    norm_groups: int
    logit_scale: float
    layers: List[dict]
    params_dtype: torch.dtype = torch.bfloat16
    max_position_embeddings: Optional[int] = None   # no position enters the model: no limit
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, dtype=torch.bfloat16) -> "BezuraxConfig":
        norm = d["norm"]
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(norm["eps"]),
                   norm_groups=int(norm.get("groups", 1)), logit_scale=float(d.get("logit_scale", 1.0)),
                   layers=list(d["layers"]), params_dtype=dtype, raw=d)

    def owner(self, i: int) -> int:
        """the layer whose weights layer i uses"""
        seen = set()
        while self.layers[i].get("weights_of") is not None:
            if i in seen:
                raise ValueError(f"layers share weights in a circle at layer {i}")
            seen.add(i)
            i = int(self.layers[i]["weights_of"])
        return i


class BezuraxBlock(nn.Module):
    """Weights of one layer: two norm weights, the parallel mixer, the experts."""

    def __init__(self, cfg: BezuraxConfig, spec: dict, decay_rank: int):
        super().__init__()
        W, dt, eps = cfg.hidden_size, cfg.params_dtype, cfg.norm_eps
        if spec["type"] != "parallel":
            raise ValueError(f"unknown mixer type {spec['type']!r}")
        m = spec["mixer"]
        lf, rt = m["left"], m["right"]
        mask = lf["mask"]
        left = PooledWindowAttention(W, int(lf["heads"]), int(lf["kv_heads"]), int(lf["dim"]), int(lf["vdim"]),
                                     float(lf["scale"]), int(mask["size"]), int(mask["pool"]), eps,
                                     values_are_keys=True, own_projections=False, dtype=dt)
        right = DeltaRuleMixer(W, int(rt["heads"]), int(rt["dim"]), decay_rank, eps, own_projections=False, dtype=dt)
        self.norm1 = nn.Parameter(torch.ones(W, dtype=torch.float32))
        self.mixer = ParallelMixer(W, left, right, float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)),
                                   dtype=dt)
        mlp = spec.get("mlp")
        if mlp:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            ro, ex, sh = mlp["router"], mlp["expert"], mlp.get("shared")
            gr = ro.get("groups") or {}
            self.norm2 = nn.Parameter(torch.ones(W, dtype=torch.float32))
            self.mlp = RoutedExpertsMLP(
                W, int(ro["experts"]), int(ro["top"]), int(ex["ff"]), float(ex["limit"]),
                groups=int(gr.get("count", 1)), keep=int(gr.get("keep", gr.get("count", 1))),
                route_scale=float(ro.get("scale", 1.0)), shared_ff=int(sh["ff"]) if sh else None,
                shared_limit=float(sh["limit"]) if sh else None, dtype=dt)
        else:
            self.norm2, self.mlp = None, None


class BezuraxModel(nn.Module):
    ragged_batch = True                 # the engine schedules mixed prefill/decode steps for this model
    native_extensions = ("hybrid",)     # what a serving process has to build for it (ops/ragged.py)

    def __init__(self, config: BezuraxConfig, decay_ranks: Optional[Dict[int, int]] = None):
        super().__init__()
        self.config = config
        W, dt = config.hidden_size, config.params_dtype
        self.embedding = nn.Parameter(torch.zeros(config.vocab_size, W, dtype=dt))   # also the output matrix
        self.blocks = nn.ModuleDict()
        for i, spec in enumerate(config.layers):
            if config.owner(i) == i:
                rank = (decay_ranks or {}).get(i, int(spec["mixer"]["right"].get("decay_rank", 16)))
                self.blocks[str(i)] = BezuraxBlock(config, spec, rank)
        for i in range(config.num_layers):
            if str(config.owner(i)) not in self.blocks:
                raise ValueError(f"layer {i} uses the weights of layer {config.owner(i)}, which has none of its own")
        self.final_norm_weight = nn.Parameter(torch.ones(W, dtype=torch.float32))
        self.layer_trace: Optional[list] = None   # debugging: residual stream after every layer

    def block_of(self, i: int) -> BezuraxBlock:
        return self.blocks[str(self.config.owner(i))]

    # -- what the cache/state manager must provide ------------------------------

    def inference_spec(self, page: int = 64) -> InferenceSpec:
        caches, states = {}, {}
        for i in range(self.config.num_layers):
            mixer = self.block_of(i).mixer
            caches.update(mixer.cache_spec(f"l{i}", page))
            states.update(mixer.state_spec(f"l{i}"))
        return InferenceSpec(caches, states)

    # -- forward ------------------------------------------------------------------

    def forward_ragged(self, tokens: torch.Tensor, ctx, want: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tokens [T] laid out by ctx.batch -> logits fp32 [len(want) or T, vocab]."""
        cfg = self.config
        dt, groups, eps = cfg.params_dtype, cfg.norm_groups, cfg.norm_eps
        x = R.embed_plain(tokens, self.embedding)                  # [T, W] fp32 residual
        y = None
        for i in range(cfg.num_layers):
            blk = self.block_of(i)
            h1, h2 = R.residual_group_norm(x, y, blk.norm1, blk.norm2, groups, eps, dt)
            y = blk.mixer(h1, ctx, f"l{i}")
            if blk.mlp is not None:
                y = blk.mlp(h2, add=y)
            if self.layer_trace is not None:
                x.add_(y.float())
                y = None
                self.layer_trace.append(x.clone())
        h, _ = R.residual_group_norm(x, y, self.final_norm_weight, None, groups, eps, dt)
        if want is not None:
            h = h.index_select(0, want)
        return F.linear(h, self.embedding).float() * cfg.logit_scale

    def forward(self, input_ids: torch.Tensor, inference_context=None, want=None) -> torch.Tensor:
        """[b, s] ids -> logits [s, b, vocab] from empty caches and states (the
        call shape of the framework's other causal LMs); with an
        inference_context whose batch is laid out, ids are the flat tokens."""
        if inference_context is not None:
            return self.forward_ragged(input_ids.reshape(-1), inference_context, want)
        from megatron_amd.inference.contexts import HybridInferenceContext

        b, s = input_ids.shape
        bs = 64
        spec = self.inference_spec(bs)
        per = (s + bs - 1) // bs
        ctx = HybridInferenceContext(spec.caches, spec.states, b * per, bs, b,
                                     dtype=self.config.params_dtype, device=input_ids.device)
        tables = [ctx.allocator.allocate(per) for _ in range(b)]
        ctx.begin_batch([s] * b, [0] * b, [ctx.acquire_slot() for _ in range(b)], tables)
        logits = self.forward_ragged(input_ids.reshape(-1), ctx)
        return logits.view(b, s, -1).transpose(0, 1)


# ---------------------------------------------------------------------------
# weights: checkpoint tensor names -> module parameters
# ---------------------------------------------------------------------------


def decay_ranks_of(cfg: BezuraxConfig, shapes: Dict[str, tuple]) -> Dict[int, int]:
    """The decay bottleneck's size is given by its tensor's shape alone."""
    return {i: int(shapes[f"l{i}.mix.right.w1"][0]) for i in range(cfg.num_layers) if cfg.owner(i) == i}


def load_bezurax_state(model: BezuraxModel, tensors: Dict[str, torch.Tensor]) -> None:
    """Copy a checkpoint's tensors (name -> tensor, Linear weights [out, in])
    into the model, fusing the projections that run as one GEMM."""
    used = set()

    def get(name):
        used.add(name)
        return tensors[name]

    with torch.no_grad():
        model.embedding.data.copy_(get("embed"))
        for key, blk in model.blocks.items():
            p = f"l{key}."
            blk.norm1.data.copy_(get(p + "norm1"))
            mx, lf, rt = blk.mixer, blk.mixer.left, blk.mixer.right
            a, b = p + "mix.left.", p + "mix.right."
            mx.w_in.data.copy_(torch.cat([get(a + "q"), get(a + "k"), get(b + "r"), get(b + "k"), get(b + "v"),
                                          get(b + "g"), get(b + "a"), get(b + "w1")], dim=0))
            mx.w_out.data.copy_(torch.cat([get(a + "o"), get(b + "o")], dim=1))
            lf.q_norm.data.copy_(get(a + "q.norm"))
            lf.k_norm.data.copy_(get(a + "k.norm"))
            rt.w2.data.copy_(get(b + "w2"))
            rt.w0.data.copy_(get(b + "w0"))
            rt.a_bias.data.copy_(get(b + "a.b"))
            rt.norm_weight.data.copy_(get(b + "norm"))
            if blk.mlp is not None:
                ff, q = blk.mlp, p + "mlp."
                blk.norm2.data.copy_(get(p + "norm2"))
                rows = [get(q + "router")] + ([get(q + "shared.sg")] if ff.shared_ff else [])
                ff.w_router.data.copy_(torch.cat(rows, dim=0))
                for e in range(ff.experts):
                    ff.w_gate_up.data[e].copy_(torch.cat([get(f"{q}e{e}.gate"), get(f"{q}e{e}.up")], dim=0))
                    ff.w_down.data[e].copy_(get(f"{q}e{e}.down"))
                if ff.shared_ff:
                    ff.ws_gate_up.data.copy_(torch.cat([get(q + "shared.gate"), get(q + "shared.up")], dim=0))
                    ff.ws_down.data.copy_(get(q + "shared.down"))
        model.final_norm_weight.data.copy_(get("final.norm"))
    unused = set(tensors) - used
    if unused:
        import warnings

        warnings.warn(f"checkpoint tensors without a place in the model are ignored: {sorted(unused)[:8]}")


def build_bezurax_from_dir(path: str, dtype=torch.bfloat16, device="cpu") -> BezuraxModel:
    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        cfg = BezuraxConfig.from_dict(json.load(f), dtype=dtype)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    model = BezuraxModel(cfg, decay_ranks_of(cfg, {k: tuple(v.shape) for k, v in tensors.items()}))
    load_bezurax_state(model, tensors)
    return model.to(device).eval()
