"""Bezutar: a decoder-only LM that stacks, in any order given by its
config.json, latent attention with a softmax sink (optionally reading another
layer's cache), mLSTM and minGRU mixers, each behind a residual causal
convolution, with xIELU feed-forwards, several hyper-connected residual
streams, and a token + hashed-bigram + learned-position embedding.

The model only has a ragged forward: a flat batch of tokens laid out by the
engine's cache/state manager (HybridInferenceContext.begin_batch).  Whole
sequences, portions of prompts and single decoded tokens are the same path;
``forward(input_ids)`` wraps it for [b, s] inputs with a throw-away context.

Everything is read from config.json: sizes, layer order, constants; optional
sections (streams, canon, embedding.bigram, rot.scaling, mlp) may be absent.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R
from megatron_amd.ssm.mingru import MinGRUMixer
from megatron_amd.ssm.mlstm import MLSTMMixer
from megatron_amd.transformer.canon import CanonConv
from megatron_amd.transformer.hyper_connections import HyperConnection
from megatron_amd.transformer.latent_sink_attention import LatentSinkAttention
from megatron_amd.transformer.mlp import XieluMLP


@dataclass
class BezutarConfig:
    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    norm_eps: float
    layers: List[dict]
    streams: Optional[int] = None          # None: one plain residual stream
    canon_taps: Optional[int] = None       # None: no input convolution
    bigram: Optional[dict] = None          # buckets, mul_prev, mul_cur
    params_dtype: torch.dtype = torch.bfloat16
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, dtype=torch.bfloat16) -> "BezutarConfig":
        return cls(
            vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
            max_position_embeddings=int(d["max_positions"]),
            norm_eps=float(d["norm"]["eps"]), layers=list(d["layers"]),
            streams=int(d["streams"]) if d.get("streams") else None,
            canon_taps=int(d["canon"]["taps"]) if d.get("canon") else None,
            bigram=(d.get("embedding") or {}).get("bigram"),
            params_dtype=dtype, raw=d)


@dataclass
class InferenceSpec:
    """What a model asks of the cache/state manager: paged pools (name -> row
    width, or (row width, rows a page) for pools that hold fewer rows than
    tokens) and per-request state tensors (name -> (shape, dtype))."""

    caches: Dict[str, int]
    states: Dict[str, tuple]


class _Sublayer(nn.Module):
    """norm weight + hyper-connection + the function between them."""

    def __init__(self, hidden: int, streams: int):
        super().__init__()
        self.norm_weight = nn.Parameter(torch.zeros(hidden, dtype=torch.float32))  # applied as 1 + w
        self.hc = HyperConnection(streams)


class BezutarLayer(nn.Module):
    def __init__(self, cfg: BezutarConfig, index: int):
        super().__init__()
        spec = cfg.layers[index]
        m = spec["mixer"]
        W, dt, S = cfg.hidden_size, cfg.params_dtype, cfg.streams or 1
        self.kind = spec["type"]
        self.sub1 = _Sublayer(W, S)
        self.canon = CanonConv(W, cfg.canon_taps, f"l{index}.canon") if cfg.canon_taps else None
        if self.kind == "latent_attention":
            src = m.get("kv_from")
            rot = m["rot"]
            self.mixer = LatentSinkAttention(
                W, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"],
                float(m["scale"]), int(rot["dims"]), float(rot["base"]), rot.get("scaling"),
                cfg.norm_eps, cfg.max_position_embeddings,
                cache_name=f"l{index if src is None else int(src)}.latent", owns_cache=src is None, dtype=dt)
        elif self.kind == "mlstm":
            self.mixer = MLSTMMixer(W, m["heads"], m["dim"], m["vdim"], float(m["gate_cap"]),
                                    cfg.norm_eps, f"l{index}.mlstm", dtype=dt)
        elif self.kind == "mingru":
            self.mixer = MinGRUMixer(W, m["width"], f"l{index}.mingru", dtype=dt)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        if mlp:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            self.sub2 = _Sublayer(W, S)
            self.mlp = XieluMLP(W, mlp["ff"], dtype=dt)
        else:
            self.sub2, self.mlp = None, None

    def sublayers(self):
        yield self.sub1, self._mix
        if self.mlp is not None:
            yield self.sub2, self._ff

    def _mix(self, h, ctx, dt):
        h = self.canon(h, ctx, dt) if self.canon is not None else h.to(dt)
        return self.mixer(h, ctx)

    def _ff(self, h, ctx, dt):
        return self.mlp(h.to(dt))


class BezutarModel(nn.Module):
    ragged_batch = True   # the engine schedules mixed prefill/decode steps for this model

    def __init__(self, config: BezutarConfig):
        super().__init__()
        self.config = config
        W, dt = config.hidden_size, config.params_dtype
        self.embedding = nn.Parameter(torch.zeros(config.vocab_size, W, dtype=dt))
        self.bigram = (nn.Parameter(torch.zeros(config.bigram["buckets"] + 1, W, dtype=dt))
                       if config.bigram else None)
        self.position = nn.Parameter(torch.zeros(config.max_position_embeddings, W, dtype=dt))
        self.layers = nn.ModuleList([BezutarLayer(config, i) for i in range(config.num_layers)])
        self.final_norm_weight = nn.Parameter(torch.zeros(W, dtype=torch.float32))
        self.output_weight = nn.Parameter(torch.zeros(config.vocab_size, W, dtype=dt))
        S = config.streams or 1
        self.register_buffer("_ones", torch.ones(S, dtype=torch.float32), persistent=False)
        self.layer_trace: Optional[list] = None   # debugging: sum of streams after every layer

    # -- what the cache/state manager must provide ------------------------------

    def inference_spec(self, page: int = 64) -> InferenceSpec:
        caches, states = {}, {}
        for layer in self.layers:
            caches.update(layer.mixer.cache_spec())
            states.update(layer.mixer.state_spec())
            if layer.canon is not None:
                states.update(layer.canon.state_spec())
        if self.bigram is not None:
            states["embed.prev"] = ((), torch.int32)
        return InferenceSpec(caches, states)

    # -- forward ------------------------------------------------------------------

    def forward_ragged(self, tokens: torch.Tensor, ctx, want: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tokens [T] laid out by ctx.batch -> logits fp32 [len(want) or T, vocab]."""
        cfg = self.config
        dt = cfg.params_dtype
        batch = ctx.batch
        bg = cfg.bigram or {}
        x = R.embed_tokens(tokens, batch, self.embedding, self.bigram, self.position,
                           ctx.states.get("embed.prev"), bg.get("mul_prev", 0), bg.get("mul_cur", 0),
                           bg.get("buckets", 1))
        S = cfg.streams or 1
        streams = x.unsqueeze(1).expand(-1, S, -1).contiguous()      # [T, S, W] fp32
        y, prev = None, None
        for layer in self.layers:
            for sub, fn in layer.sublayers():
                h = R.hc_mix_norm(streams, y, prev.mix if prev is not None else None,
                                  prev.write if prev is not None else None,
                                  sub.hc.read, sub.norm_weight, cfg.norm_eps)
                y = fn(h, ctx, dt)
                prev = sub.hc
            if self.layer_trace is not None:
                R.hc_mix_norm(streams, y, prev.mix, prev.write, None, None, cfg.norm_eps)
                y, prev = None, None
                self.layer_trace.append(streams.sum(dim=1))
        h = R.hc_mix_norm(streams, y, prev.mix if prev is not None else None,
                          prev.write if prev is not None else None,
                          self._ones, self.final_norm_weight, cfg.norm_eps)
        if want is not None:
            h = h.index_select(0, want)
        return F.linear(h.to(dt), self.output_weight).float()

    def forward(self, input_ids: torch.Tensor, inference_context=None, want=None) -> torch.Tensor:
        """[b, s] ids -> logits [s, b, vocab] from empty caches and states (the
        call shape of the framework's other causal LMs); with an
        inference_context whose batch is laid out, ids are the flat tokens."""
        if inference_context is not None:
            return self.forward_ragged(input_ids.reshape(-1), inference_context, want)
        from megatron_amd.inference.contexts import HybridInferenceContext

        b, s = input_ids.shape
        spec = self.inference_spec()
        bs = 64
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


def _load_mixer(layer: BezutarLayer, get, p: str):
    mx = layer.mixer
    if layer.kind == "latent_attention":
        parts = [get(p + "dq")]
        if mx.owns_cache:
            parts.append(get(p + "dkv"))
            mx.kv_norm.data.copy_(get(p + "dkv.norm"))
        parts.append(get(p + "g"))
        mx.w_in.data.copy_(torch.cat(parts, dim=0))
        mx.q_norm.data.copy_(get(p + "dq.norm"))
        mx.w_uq.data.copy_(get(p + "uq"))
        mx.w_uk.data.copy_(get(p + "uk").view(mx.heads, mx.dim, mx.kv_rank))
        mx.w_uv.data.copy_(get(p + "uv").view(mx.heads, mx.vdim, mx.kv_rank))
        mx.sink.data.copy_(get(p + "sink"))
        mx.w_out.data.copy_(get(p + "o"))
    elif layer.kind == "mlstm":
        mx.w_in.data.copy_(torch.cat([get(p + "q"), get(p + "k"), get(p + "v"), get(p + "g")], dim=0))
        mx.w_gates.data.copy_(torch.cat([get(p + "i"), get(p + "f")], dim=0))
        mx.bias_i.data.copy_(get(p + "i.b"))
        mx.bias_f.data.copy_(get(p + "f.b"))
        mx.norm_weight.data.copy_(get(p + "norm"))
        mx.w_out.data.copy_(get(p + "o"))
    else:
        mx.w_in.data.copy_(torch.cat([get(p + "z"), get(p + "x"), get(p + "g")], dim=0))
        mx.bias_z.data.copy_(get(p + "z.b"))
        mx.bias_x.data.copy_(get(p + "x.b"))
        mx.w_out.data.copy_(get(p + "o"))


def load_bezutar_state(model: BezutarModel, tensors: Dict[str, torch.Tensor]) -> None:
    """Copy a checkpoint's tensors (name -> tensor, Linear weights [out, in])
    into the model, fusing the projections that run as one GEMM."""
    used = set()

    def get(name):
        used.add(name)
        return tensors[name]

    cfg = model.config
    with torch.no_grad():
        model.embedding.data.copy_(get("embed"))
        if model.bigram is not None:
            model.bigram.data.copy_(get("bigram"))
        if "pos" in tensors:
            model.position.data.copy_(get("pos"))
        else:
            model.position = None       # no learned position table in this checkpoint
        for i, layer in enumerate(model.layers):
            p = f"l{i}."
            subs = [(layer.sub1, 1)] + ([(layer.sub2, 2)] if layer.sub2 is not None else [])
            for sub, q in subs:
                sub.norm_weight.data.copy_(get(p + f"norm{q}"))
                if cfg.streams:
                    sub.hc.read.data.copy_(get(p + f"hc{q}.in"))
                    sub.hc.write.data.copy_(get(p + f"hc{q}.out"))
                    sub.hc.mix.data.copy_(get(p + f"hc{q}.mix"))
            if layer.canon is not None:
                layer.canon.weight.data.copy_(get(p + "canon1"))
            _load_mixer(layer, get, p + "mix.")
            if layer.mlp is not None:
                layer.mlp.w_up.data.copy_(get(p + "mlp.up"))
                layer.mlp.w_down.data.copy_(get(p + "mlp.down"))
                layer.mlp.act.data.copy_(get(p + "mlp.act"))
        model.final_norm_weight.data.copy_(get("final.norm"))
        model.output_weight.data.copy_(get("head"))
    unused = set(tensors) - used
    if unused:
        import warnings

        warnings.warn(f"checkpoint tensors without a place in the model are ignored: {sorted(unused)[:8]}")


def build_bezutar_from_dir(path: str, dtype=torch.bfloat16, device="cpu") -> BezutarModel:
    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        cfg = BezutarConfig.from_dict(json.load(f), dtype=dtype)
    model = BezutarModel(cfg)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    load_bezutar_state(model, tensors)
    return model.to(device).eval()
