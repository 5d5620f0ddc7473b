"""Ragged-batch sequence ops: embedding with hashed bigrams, hyper-connection
stream mixing fused with RMS norm, residual causal convolution with carried
taps, minGRU and mLSTM recurrences with per-request state slots, latent-cache
attention with a softmax sink, xIELU.

Dispatch rule (same as megatron_amd.ops): tensors on a HIP device run the
CDNA4 kernels of the ``_ragged_ops`` extension (csrc/ragged/*.hip) and RAISE
when it is not built; CPU tensors run the torch implementations in
``ragged_reference`` so every path tests without a GPU.
MEGATRON_AMD_FORCE_REFERENCE=1 forces the torch path (numerics tests).
"""

from __future__ import annotations

import os
from typing import Optional

import torch

from megatron_amd.ops import ragged_reference as ref
from megatron_amd.ops.ragged_reference import rope_table  # noqa: F401  (host-side table)

_C = None
_IMPORT_ERROR: Optional[str] = None


def _load():
    global _C, _IMPORT_ERROR
    if _C is not None:
        return _C
    try:
        from megatron_amd.ops import _ragged_ops as mod  # built in-tree (setup.py / build_ragged_ops)

        _C = mod
    except Exception as e:  # noqa: BLE001
        _IMPORT_ERROR = repr(e)
    return _C


_load()


def build_ragged_ops(verbose: bool = False) -> None:
    """Compile ONLY the ragged-ops extension in-tree (a serving process of a
    model that needs nothing else calls this on first use)."""
    import subprocess
    import sys

    repo = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = dict(os.environ, MEGATRON_AMD_ONLY_EXT="ragged", PYTORCH_ROCM_ARCH="gfx950")
    env.setdefault("MAX_JOBS", "8")
    out = None if verbose else subprocess.DEVNULL
    subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"], cwd=repo, env=env,
                   check=True, stdout=sys.stderr if verbose else out, stderr=sys.stderr if verbose else out)
    if _load() is None:
        raise RuntimeError(f"ragged ops extension did not import after build: {_IMPORT_ERROR}")


def has_native() -> bool:
    return _C is not None and os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") != "1"


def _native(x: torch.Tensor) -> bool:
    if not x.is_cuda:
        return False
    if os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") == "1":
        return False
    if _C is None:
        raise RuntimeError(
            "megatron_amd ragged-ops HIP extension not built but a GPU tensor hit the ops layer "
            f"(import error: {_IMPORT_ERROR}). Run megatron_amd.ops.ragged.build_ragged_ops().")
    return True


_EMPTY = {}


def _none(device):
    t = _EMPTY.get(device)
    if t is None:
        t = _EMPTY[device] = torch.empty(0, device=device)
    return t


def embed_tokens(tokens, batch, embed, bigram, pos, prev_state, mul_prev=0, mul_cur=0, buckets=1):
    if _native(embed):
        d = embed.device
        return _C.embed_tokens(tokens, batch.cu_tokens, batch.slots, batch.tok_req, batch.tok_pos,
                               embed, bigram if bigram is not None else _none(d),
                               pos if pos is not None else _none(d),
                               prev_state if prev_state is not None else _none(d),
                               int(mul_prev), int(mul_cur), int(buckets))
    return ref.embed_tokens(tokens, batch, embed, bigram, pos, prev_state, mul_prev, mul_cur, buckets)


def hc_mix_norm(streams, y, mix, out_w, in_w, norm_w, eps):
    if _native(streams):
        d = streams.device
        h = _C.hc_mix_norm(streams, y if y is not None else _none(d),
                           mix if y is not None else _none(d), out_w if y is not None else _none(d),
                           in_w if in_w is not None else _none(d),
                           norm_w if in_w is not None else _none(d), float(eps))
        return h if in_w is not None else None
    return ref.hc_mix_norm(streams, y, mix, out_w, in_w, norm_w, eps)


def canon_conv(h, weight, state, batch, out_dtype):
    if _native(h):
        return _C.canon_conv(h, weight, state, batch.cu_tokens, batch.slots, batch.tok_req,
                             out_dtype == torch.bfloat16)
    return ref.canon_conv(h, weight, state, batch, out_dtype)


def mingru_scan(zxg, bias_z, bias_x, state, batch, out_dtype):
    if _native(zxg):
        return _C.mingru_scan(zxg, bias_z, bias_x, state, batch.cu_tokens, batch.slots)
    return ref.mingru_scan(zxg, bias_z, bias_x, state, batch, out_dtype)


def mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, cap, eps,
               state_S, state_n, state_m, batch, out_dtype):
    if _native(qkvg):
        return _C.mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, float(cap), float(eps),
                             state_S, state_n, state_m, batch.cu_tokens, batch.slots)
    return ref.mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, cap, eps,
                          state_S, state_n, state_m, batch, out_dtype)


def latent_kv_store(dkv, norm_w, eps, cos, sin, rot_dims, rank, pool, batch):
    if _native(dkv):
        _C.latent_kv_store(dkv, norm_w, float(eps), cos, sin, int(rot_dims), int(rank), pool,
                           batch.tok_pos, batch.tok_row)
        return
    ref.latent_kv_store(dkv, norm_w, eps, cos, sin, rot_dims, rank, pool, batch)


def latent_q_prepare(dq, norm_w, eps, out_dtype):
    if _native(dq):
        return _C.rmsnorm_rows(dq, norm_w, float(eps))
    return ref.latent_q_prepare(dq, norm_w, eps, out_dtype)


def assemble_latent_q(q_abs, q_rot, cos, sin, rot_dims, batch):
    """[absorbed unrotated part | rotated part after RoPE] -> [T, H, rank + rot]."""
    if _native(q_abs):
        return _C.assemble_latent_q(q_abs, q_rot, cos, sin, int(rot_dims), batch.tok_pos)
    return torch.cat([q_abs, ref.rope_heads(q_rot, cos, sin, rot_dims, batch)], dim=-1)


def _mfma_ok(q, rank) -> bool:
    Dk = q.shape[2]
    return (q.dtype == torch.bfloat16 and Dk % 8 == 0 and rank % 4 == 0 and Dk <= 576 and rank <= 512
            and os.environ.get("MEGATRON_AMD_NO_MFMA_LATENT", "0") != "1")


def latent_sink_attention(q, pool, rank, sink, scale, batch):
    """[T, H, rank] (a view of an [H, T, rank] buffer on the kernel paths)."""
    if _native(q):
        if _mfma_ok(q, rank):
            # matrix-core kernel: 64 (token, head) rows per workgroup; steps with few
            # rows and long contexts (decode) also split the keys over workgroups
            tiles = batch.row_tiles(q.shape[1], q.device)
            nblk = tiles.shape[0]
            nsplit = max(1, min((batch.max_context + 63) // 64, 1024 // nblk, 64))
            return _C.latent_sink_attention_mfma(q, pool, int(rank), sink, float(scale), tiles, batch.cu_tokens,
                                                 batch.start_pos, batch.block_tables, int(batch.block_size),
                                                 int(nsplit))
        return _C.latent_sink_attention(q, pool, int(rank), sink, float(scale), batch.tok_req,
                                        batch.tok_pos, batch.block_tables, int(batch.block_size))
    return ref.latent_sink_attention(q, pool, rank, sink, scale, batch)


def xielu(z, act, out_dtype):
    if _native(z):
        return _C.xielu(z, act)
    return ref.xielu(z, act, out_dtype)


def gate_heads(x, gate_pre, heads):
    if _native(x):
        return _C.gate_heads(x, gate_pre, int(heads))
    return ref.gate_heads(x, gate_pre, heads)
