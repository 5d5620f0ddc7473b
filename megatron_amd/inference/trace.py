"""Replay of given token streams through the dynamic engine, step by step.

Input: one JSON object a line,
    {"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}, ...], "end": [...]}
Every entry brings a request's next tokens; all entries of a step run as ONE
mixed batch through DynamicInferenceEngine.forward_batch (the same step
function the engine's own scheduler drives), on the caches and states earlier
steps left.  For a step that wants logits, ``<out>/<step>.f32`` receives the
rows [wanted, vocab] as little-endian fp32, in entry and ``want`` order; after
every step the line ``done <step>`` is printed.  Requests named in "end"
give their pages and state slot back after the step.  Nothing is sampled.
"""

from __future__ import annotations

import json
import os
import sys

import torch

PAGE = 64          # cache page size in tokens
SLOTS = 4          # requests that may be live at once


def build_engine(model_dir: str, dtype: torch.dtype, max_tokens: int, device=None):
    from megatron_amd.inference.engine import DynamicInferenceEngine
    from megatron_amd.models.registry import build_from_dir

    if device is None:
        device = torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")
    if dtype == torch.float32:
        # true 32-bit products: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    model = build_from_dir(model_dir, dtype=dtype, device=device)
    if not getattr(model, "ragged_batch", False):
        raise SystemExit("this model has no mixed-batch step function")
    pages = (max_tokens + PAGE - 1) // PAGE
    return DynamicInferenceEngine(model, num_blocks=pages, block_size=PAGE, max_batch=SLOTS,
                                  device=device, use_hip_graphs=False, enable_prefix_caching=False)


def replay(engine, lines, out_dir: str, log=sys.stdout) -> None:
    live = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        feeds, want = [], []
        for e in step["entries"]:
            req = live.get(e["id"])
            if req is None:
                req = live[e["id"]] = engine.open_request()
            if not e["tokens"]:
                continue                    # admitted, nothing to run yet
            feeds.append((req, [int(t) for t in e["tokens"]]))
            want.append([int(w) for w in e.get("want", [])])
        logits = engine.forward_batch(feeds, want) if feeds else None
        if logits is not None:
            data = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4")
            tmp = os.path.join(out_dir, ".%d.part" % step["step"])
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(out_dir, "%d.f32" % step["step"]))
        elif engine.device.type == "cuda":
            torch.cuda.synchronize()
        for rid in step.get("end", []):
            req = live.pop(rid, None)
            if req is not None:
                engine.close_request(req)
        log.write("done %d\n" % step["step"])
        log.flush()


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at once (each rounded up to a page)")
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)
    device = torch.device(a.device) if a.device else None
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    engine = build_engine(a.model, dtype, a.max_tokens, device)
    if engine.device.type == "cuda":
        # kernels are compiled in-tree at the first call, and only the
        # extensions this model's layers use
        from megatron_amd.ops import ragged

        ragged.ensure_built(getattr(engine.model, "native_extensions", ("ragged",)), verbose=True)
    os.makedirs(a.out, exist_ok=True)
    replay(engine, sys.stdin, a.out)
    return 0
