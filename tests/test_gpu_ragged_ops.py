"""GPU numerics of the ragged-batch HIP kernels: every kernel against the plain
torch implementation of the same op (ops/ragged_reference.py) on the same
inputs, in fp32 and bf16 storage, on a ragged batch that mixes prompt portions
with single tokens, uses non-trivial page tables and reuses state slots."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ctx(device, dtype, caches, states, counts, starts, bs=16):
    from megatron_amd.inference.contexts import HybridInferenceContext

    R = len(counts)
    pages = [(s + c + bs - 1) // bs for s, c in zip(starts, counts)]
    ctx = HybridInferenceContext(caches, states, sum(pages) + 3, bs, R + 2, dtype=dtype, device=device)
    ctx.allocator.allocate(2)                       # skew page ids
    slots = [ctx.acquire_slot() for _ in range(R + 1)][1:]
    tables = [ctx.allocator.allocate(p)[::-1] for p in pages]
    ctx.begin_batch(counts, starts, slots, tables)
    return ctx


COUNTS, STARTS = [37, 1, 5, 2], [0, 20, 30, 3]


def _both(fn, dtype):
    """Run fn on GPU (kernels) and on CPU (torch reference) with the same seed."""
    outs = []
    for dev in ("cuda", "cpu"):
        torch.manual_seed(7)
        outs.append(fn(torch.device(dev), dtype))
    return outs


def _close(a, b, dtype, what=""):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    a, b = a.float().cpu(), b.float().cpu()
    err = (a - b).abs().max().item() / max(b.abs().max().item(), 1e-6)
    assert err < tol, f"{what}: relative error {err}"


def _rand(shape, dtype, device, scale=1.0):
    return (torch.randn(shape, dtype=torch.float32) * scale).to(dtype).to(device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_and_streams(dtype):
    from megatron_amd.ops import ragged as R

    assert R.has_native(), "ragged-ops extension must be built for GPU tests"
    V, W, S, B = 50, 72, 3, 11

    def run(dev, dt):
        ctx = _ctx(dev, dt, {}, {"prev": ((), torch.int32)}, COUNTS, STARTS)
        ctx.states["prev"].copy_(torch.arange(ctx.states["prev"].numel()) + 3)
        toks = torch.randint(0, V, (sum(COUNTS),)).to(dev)
        emb, bg, pos = _rand((V, W), dt, dev), _rand((B + 1, W), dt, dev), _rand((64, W), dt, dev)
        x = R.embed_tokens(toks, ctx.batch, emb, bg, pos, ctx.states["prev"], 31, 5, B)
        streams = x.unsqueeze(1).expand(-1, S, -1).contiguous()
        mix, ow, iw = _rand((S, S), torch.float32, dev), _rand((S,), torch.float32, dev), _rand((S,), torch.float32, dev)
        nw = _rand((W,), torch.float32, dev, 0.1)
        h0 = R.hc_mix_norm(streams, None, None, None, iw, nw, 1e-5)
        y = _rand((sum(COUNTS), W), dt, dev)
        h1 = R.hc_mix_norm(streams, y, mix, ow, iw, nw, 1e-5)
        R.hc_mix_norm(streams, y, mix, ow, None, None, 1e-5)
        return x, h0, h1, streams, ctx.states["prev"].float()

    g, c = _both(run, dtype)
    for a, b, n in zip(g, c, ["embed", "pre", "mix+pre", "streams", "prev token"]):
        _close(a, b, torch.float32, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [2, 4, 7])
def test_canon_conv(dtype, taps):
    from megatron_amd.ops import ragged as R

    W = 40

    def run(dev, dt):
        ctx = _ctx(dev, dt, {}, {"c": ((taps - 1, W), torch.float32)}, COUNTS, STARTS)
        ctx.states["c"].copy_(torch.randn(ctx.states["c"].shape))
        h = _rand((sum(COUNTS), W), torch.float32, dev)
        w = _rand((W, taps), torch.float32, dev)
        return R.canon_conv(h, w, ctx.states["c"], ctx.batch, dt), ctx.states["c"].clone()

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "conv")
    _close(g[1], c[1], torch.float32, "carried taps")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mingru(dtype):
    from megatron_amd.ops import ragged as R

    C = 70

    def run(dev, dt):
        ctx = _ctx(dev, dt, {}, {"s": ((C,), torch.float32)}, COUNTS, STARTS)
        ctx.states["s"].copy_(torch.randn(ctx.states["s"].shape))
        zxg = _rand((sum(COUNTS), 3 * C), dt, dev, 2.0)
        bz, bx = _rand((C,), torch.float32, dev), _rand((C,), torch.float32, dev)
        return R.mingru_scan(zxg, bz, bx, ctx.states["s"], ctx.batch, dt), ctx.states["s"].clone()

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "out")
    _close(g[1], c[1], torch.float32, "state")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,V", [(3, 24, 40), (2, 80, 16), (1, 8, 8)])
def test_mlstm(dtype, H, D, V):
    from megatron_amd.ops import ragged as R

    def run(dev, dt):
        st = {"S": ((H, D, V), torch.float32), "n": ((H, D), torch.float32), "m": ((H,), torch.float32)}
        ctx = _ctx(dev, dt, {}, st, COUNTS, STARTS)
        for k in st:
            ctx.states[k].copy_(torch.randn(ctx.states[k].shape) * 0.3)
        T = sum(COUNTS)
        qkvg = _rand((T, 2 * H * D + 2 * H * V), dt, dev)
        gates = _rand((T, 2 * H), torch.float32, dev, 3.0)
        bi, bf = _rand((H,), torch.float32, dev), _rand((H,), torch.float32, dev) + 2
        nw = _rand((H * V,), torch.float32, dev)
        o = R.mlstm_scan(qkvg, gates, bi, bf, nw, H, D, V, 9.0, 1e-5, ctx.states["S"], ctx.states["n"],
                         ctx.states["m"], ctx.batch, dt)
        return o, ctx.states["S"].clone(), ctx.states["n"].clone(), ctx.states["m"].clone()

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "out")
    for a, b, n in zip(g[1:], c[1:], "Snm"):
        _close(a, b, torch.float32, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,rank,rd,rot", [(3, 40, 8, 8), (2, 200, 24, 16), (5, 320, 64, 64)])
def test_latent_attention(dtype, H, rank, rd, rot):
    from megatron_amd.ops import ragged as R

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"kv": rank + rd}, {}, COUNTS, STARTS)
        ctx.pools["kv"].copy_(torch.randn(ctx.pools["kv"].shape) * 0.5)
        T = sum(COUNTS)
        cos, sin = R.rope_table(128, rot, 10000.0, dict(factor=4.0, original=32, fast=8.0, slow=1.0))
        cos, sin = cos.to(dev), sin.to(dev)
        dkv = _rand((T, rank + rd + 5), dt, dev)[:, 2 : 2 + rank + rd]         # strided rows
        R.latent_kv_store(dkv, _rand((rank,), torch.float32, dev), 1e-5, cos, sin, rot, rank, ctx.pools["kv"], ctx.batch)
        qn = R.latent_q_prepare(_rand((T, 48), dt, dev), _rand((48,), torch.float32, dev), 1e-5, dt)
        q_abs = _rand((H, T, rank), dt, dev, 0.3).transpose(0, 1)
        q_rot = _rand((T, H, rd + 3), dt, dev)[..., 3:]
        q = R.assemble_latent_q(q_abs, q_rot, cos, sin, rot, ctx.batch)
        out = R.latent_sink_attention(q, ctx.pools["kv"], rank, _rand((H,), torch.float32, dev), 0.2, ctx.batch)
        gated = R.gate_heads(out, _rand((T, H), dt, dev), H)
        return ctx.pools["kv"].clone(), qn, q, out, gated

    g, c = _both(run, dtype)
    for a, b, n in zip(g, c, ["pool", "q norm", "q", "attention", "gate"]):
        _close(a, b, dtype, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_xielu(dtype):
    from megatron_amd.ops import ragged as R

    def run(dev, dt):
        z = _rand((33, 50), dt, dev, 2.0)
        return (R.xielu(z, torch.tensor([0.3, -0.7]).to(dev), dt),)

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "xielu")
