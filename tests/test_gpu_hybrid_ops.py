"""GPU numerics of the hybrid serving kernels (grouped norm on the fp32
residual, pooled-window attention, delta rule, routed experts): every kernel
against the plain torch implementation of the same op
(ops/ragged_reference.py) on the same inputs, in fp32 and bf16 storage, on a
ragged batch that mixes prompt portions with single tokens, uses skewed page
tables and reused state slots."""

import pytest
import torch

pytestmark = pytest.mark.gpu

from test_gpu_ragged_ops import _both, _close, _ctx, _rand  # noqa: E402

COUNTS, STARTS = [45, 1, 7, 2, 1], [0, 52, 30, 3, 11]


def _need():
    from megatron_amd.ops import ragged as R

    assert R._load("hybrid") is not None, "hybrid-ops extension must be built for GPU tests"
    return R


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("groups", [1, 4, 6])
def test_embed_and_group_norm(dtype, groups):
    R = _need()
    V, W = 50, 96

    def run(dev, dt):
        T = 13
        toks = torch.randint(0, V, (T,)).to(dev)
        emb = _rand((V, W), dt, dev)
        x = R.embed_plain(toks, emb)
        x0 = x.clone()
        wa, wb = _rand((W,), torch.float32, dev), _rand((W,), torch.float32, dev)
        a0, none = R.residual_group_norm(x, None, wa, None, groups, 1e-5, dt)
        assert none is None
        y = _rand((T, W), dt, dev)
        a1, b1 = R.residual_group_norm(x, y, wa, wb, groups, 1e-5, dt)
        yf = _rand((T, W), torch.float32, dev)
        a2, b2 = R.residual_group_norm(x, yf, wa, wb, groups, 1e-5, dt)
        return x0, a0, a1, b1, a2, b2, x

    g, c = _both(run, dtype)
    for a, b, n in zip(g, c, ["embed", "norm", "add+norm a", "add+norm b", "fp32 add a", "fp32 add b", "residual"]):
        _close(a, b, dtype if n.endswith((" a", " b", "norm")) else torch.float32, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 24, 24, 9, 4), (3, 3, 80, 80, 5, 1), (6, 1, 144, 144, 64, 7), (2, 2, 16, 16, 1, 3),
                                   (8, 2, 64, 64, 40, 6), (2, 1, 12, 12, 5, 2)])
@pytest.mark.parametrize("starts", [STARTS, [0, 300, 130, 3, 517]], ids=["short", "long"])
def test_pooled_window_attention(dtype, shape, starts):
    """heads, kv heads, dim, vdim, window, pool; page 16: pooled rows and windows cross pages;
    long contexts beside short ones make the bf16 kernel split the key tiles over workgroups"""
    R = _need()
    H, G, D, V, window, P = shape
    STARTS = starts
    bs = 16
    rpp = (bs + P - 1) // P

    def run(dev, dt):
        width = G * (D + V)
        ctx = _ctx(dev, dt, {"c": width, "c.pooled": (width, rpp)}, {}, COUNTS, STARTS, bs=bs)
        pool, pooled = ctx.pools["c"], ctx.pools["c.pooled"]
        pool.copy_(_rand(pool.shape, dt, dev))            # what earlier steps left (and junk in foreign pages)
        pooled.copy_(_rand(pooled.shape, dt, dev))
        # pooled rows of the blocks that earlier steps completed
        from megatron_amd.ops import ragged_reference as ref

        b = ctx.batch
        for r in range(b.num_requests):
            table = torch.as_tensor(b.host_tables[r], dtype=torch.long, device=dev)
            nblk = b.host_start[r] // P
            if nblk:
                rows = ref._rows_of(table, nblk * P, bs, dev)
                pooled[ref._rows_of(table, nblk, rpp, dev)] = pool[rows].float().view(nblk, P, -1).mean(1).to(dt)
        T = sum(COUNTS)
        proj = _rand((T, 5 + H * D + G * D), dt, dev)
        qn, kn = _rand((H * D,), torch.float32, dev), _rand((G * D,), torch.float32, dev)
        q = R.qk_norm_store(proj, 5, H * D, 5 + H * D, G * D, 5 + H * D, G * V, qn, kn, 1e-5, pool, b)
        R.pool_blocks(pool, pooled, P, rpp, b)
        out = torch.zeros(T, H * V + 7, dtype=dt, device=dev)
        R.pooled_window_attention(q * 3, pool, pooled, H, G, D, V, 0.3, window, P, rpp, b, out, 7, 0.8)
        return q, pool, pooled, out

    g, c = _both(run, dtype)
    for a, b, n in zip(g, c, ["q", "pool", "pooled", "attention"]):
        _close(a, b, dtype, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 16, 4), (2, 64, 16), (2, 96, 8), (1, 160, 5)])
def test_delta_rule(dtype, shape):
    R = _need()
    H, D, rank = shape
    HD = H * D

    def run(dev, dt):
        ctx = _ctx(dev, dt, {}, {"S": ((H, D, D), torch.float32)}, COUNTS, STARTS)
        ctx.states["S"].copy_(_rand(ctx.states["S"].shape, torch.float32, dev, 0.3))
        T = sum(COUNTS)
        proj = _rand((T, 3 + 5 * HD + rank), dt, dev)
        w2, w0 = _rand((HD, rank), torch.float32, dev), _rand((HD,), torch.float32, dev)
        ab, nw = _rand((HD,), torch.float32, dev), _rand((HD,), torch.float32, dev)
        out = torch.zeros(T, HD + 2, dtype=dt, device=dev)
        R.delta_rule_scan(proj, 3, 3 + HD, 3 + 2 * HD, 3 + 3 * HD, 3 + 4 * HD, 3 + 5 * HD, rank, w2, w0, ab, nw,
                          H, D, 1e-5, ctx.states["S"], ctx.batch, out, 2, 1.1)
        return out, ctx.states["S"]

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "delta rule output")
    _close(g[1], c[1], torch.float32 if dtype == torch.float32 else dtype, "delta rule state")


@pytest.mark.parametrize("cfg", [(15, 4, 5, 3), (8, 2, 1, 1), (16, 1, 8, 2), (6, 3, 6, 4), (64, 8, 8, 4)])
def test_moe_route(cfg):
    R = _need()
    E, top, groups, keep = cfg

    def run(dev, dt):
        logits = (_rand((37, E + 1), torch.float32, dev) * 2).contiguous()
        ids, w = R.moe_route(logits, E, top, groups, keep, 1.25)
        order = ids.long().argsort(dim=1)                 # compare as sets: sort by expert id
        return ids.long().gather(1, order).float(), w.gather(1, order)

    g, c = _both(run, torch.float32)
    assert torch.equal(g[0].cpu(), c[0]), "chosen experts"
    _close(g[1], c[1], torch.float32, "weights")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [40, 36])
def test_glu_and_combine(dtype, W):
    R = _need()

    def run(dev, dt):
        T, K, F_ = 9, 3, 24
        gu = _rand((T * K, 2 * F_), dt, dev, 2.0)
        y = R.clamped_glu(gu, 1.25, 1.702, dt)
        down = _rand((T * K, W), dt, dev)
        inv = torch.randperm(T * K).view(T, K).to(torch.int32).to(dev)
        w = _rand((T, K), torch.float32, dev).abs()
        sh, gate, add = _rand((T, W), dt, dev), _rand((T,), torch.float32, dev), _rand((T, W), dt, dev)
        return (y, R.moe_combine(down, inv, w, sh, gate, add), R.moe_combine(down, inv, w, None, None, None),
                R.moe_combine(down, inv, w, None, None, add))

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "glu")
    for a, b in zip(g[1:], c[1:]):
        _close(a, b, torch.float32, "combine")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_expert_pairs(dtype):
    R = _need()

    def run(dev, dt):
        T, K, W, F_, E = 5, 3, 72, 40, 6
        h = _rand((T, W), dt, dev)
        ids = torch.stack([torch.randperm(E)[:K] for _ in range(T)]).to(torch.int32).to(dev)
        wgu, wd = _rand((E, 2 * F_, W), dt, dev, 0.2), _rand((E, W, F_), dt, dev, 0.2)
        return (R.expert_pairs(h, ids, wgu, wd, 1.2, 1.702),)

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "expert pairs")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cfg", [(15, 4, 5, 3, 1), (8, 2, 1, 1, 0), (64, 8, 8, 4, 1), (5, 5, 1, 1, 2)])
def test_moe_router_fused(dtype, cfg):
    R = _need()
    E, top, groups, keep, extra = cfg

    def run(dev, dt):
        h = _rand((23, 88), dt, dev)
        wr = _rand((E + extra, 88), torch.float32, dev, 0.4)
        ids, w, ex = R.moe_router(h, wr, E, top, groups, keep, 1.25)
        order = ids.long().argsort(dim=1)
        return ids.long().gather(1, order).float(), w.gather(1, order), ex

    g, c = _both(run, dtype)
    assert torch.equal(g[0].cpu(), c[0]), "chosen experts"
    _close(g[1], c[1], torch.float32, "weights")
    if extra:
        _close(g[2], c[2], torch.float32, "extra logits")
