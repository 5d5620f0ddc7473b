"""Bezurax model family: the framework's ragged engine path against a plain
per-sequence oracle (tests/bezurax_oracle.py) on small random configurations.

Covers each mechanism alone, prefill against token-by-token decoding, prompt
portions down to two tokens, mixed batches against each request alone, reuse
of freed pages and state slots, keys far away / at page borders / just inside
and just outside the window and the pooled blocks (in prompts and in
decoding, with a peaked softmax so that one key too many or too few shows),
the first tokens of a sequence, long decoding, degenerate and unequal sizes,
weight sharing between layers, and greedy generation through the engine's own
scheduler.
"""

import copy
import math

import pytest
import torch

import bezurax_oracle as O
from megatron_amd.inference import DynamicInferenceEngine, SamplingParams
from megatron_amd.inference.contexts import HybridInferenceContext
from megatron_amd.models.bezurax import BezuraxConfig, BezuraxModel, decay_ranks_of, load_bezurax_state


def layer(heads=4, kv=2, dim=6, window=7, pool=3, scale=0.5, rheads=2, rdim=5, experts=6, top=2, ff=10,
          groups=(3, 2), shared=12, mlp=True, left_scale=0.7, right_scale=1.2, weights_of=None):
    spec = dict(type="parallel",
                mixer=dict(left=dict(heads=heads, kv_heads=kv, dim=dim, vdim=dim, scale=scale,
                                     mask=dict(size=window, pool=pool)),
                           right=dict(heads=rheads, dim=rdim), left_scale=left_scale, right_scale=right_scale),
                mlp=None)
    if mlp:
        router = dict(experts=experts, top=top, scale=1.3)
        if groups:
            router["groups"] = dict(count=groups[0], keep=groups[1])
        spec["mlp"] = dict(kind="moe", expert=dict(ff=ff, limit=1.2), router=router)
        if shared:
            spec["mlp"]["shared"] = dict(ff=shared, limit=0.9)
    if weights_of is not None:
        spec["weights_of"] = weights_of
    return spec


def make_config(layers, width=24, vocab=41, groups=3, eps=1e-5, logit_scale=1.7):
    return dict(architecture="Bezurax", vocab=vocab, width=width, norm=dict(eps=eps, groups=groups),
                logit_scale=logit_scale, layers=copy.deepcopy(layers))


def make_weights(cfg, seed=0, gain=1.0, decay_rank=3):
    """Random checkpoint tensors under the checkpoint's names (bf16-representable
    values so that both sides read the same numbers)."""
    g = torch.Generator().manual_seed(seed)
    W, out = cfg["width"], {}

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16).float()

    def lin(o, i):
        return rnd(o, i, scale=gain / math.sqrt(i))

    out["embed"] = rnd(cfg["vocab"], W)
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, lf, rt = f"l{i}.", L["mixer"]["left"], L["mixer"]["right"]
        out[p + "norm1"] = 1 + rnd(W, scale=0.2)
        a, b = p + "mix.left.", p + "mix.right."
        qw, kw, hd = lf["heads"] * lf["dim"], lf["kv_heads"] * lf["dim"], rt["heads"] * rt["dim"]
        out[a + "q"], out[a + "k"] = lin(qw, W), lin(kw, W)
        out[a + "q.norm"], out[a + "k.norm"] = 1 + rnd(qw, scale=0.2), 1 + rnd(kw, scale=0.2)
        out[a + "o"] = lin(W, lf["heads"] * lf["vdim"])
        for n in "rkvga":
            out[b + n] = lin(hd, W)
        out[b + "a.b"], out[b + "w0"] = rnd(hd, scale=0.5), rnd(hd) - 1.0
        out[b + "w1"], out[b + "w2"] = lin(decay_rank, W), rnd(hd, decay_rank)
        out[b + "norm"], out[b + "o"] = 1 + rnd(hd, scale=0.2), lin(W, hd)
        if L.get("mlp"):
            m, q = L["mlp"], p + "mlp."
            out[p + "norm2"] = 1 + rnd(W, scale=0.2)
            out[q + "router"] = lin(m["router"]["experts"], W) * 3
            for e in range(m["router"]["experts"]):
                ff = m["expert"]["ff"]
                out[f"{q}e{e}.gate"], out[f"{q}e{e}.up"], out[f"{q}e{e}.down"] = lin(ff, W) * 2, lin(ff, W) * 2, lin(W, ff)
            if m.get("shared"):
                sf = m["shared"]["ff"]
                out[q + "shared.gate"], out[q + "shared.up"], out[q + "shared.down"] = lin(sf, W) * 2, lin(sf, W), lin(W, sf)
                out[q + "shared.sg"] = lin(1, W)
    out["final.norm"] = 1 + rnd(W, scale=0.2)
    return {k: v.to(torch.bfloat16).float() for k, v in out.items()}


def build(cfg, weights, dtype=torch.float32, device="cpu"):
    c = BezuraxConfig.from_dict(cfg, dtype=dtype)
    model = BezuraxModel(c, decay_ranks_of(c, {k: tuple(v.shape) for k, v in weights.items()}))
    load_bezurax_state(model, weights)
    return model.to(device).eval()


def engine_for(model, pages=40, page=8, slots=4, **kw):
    return DynamicInferenceEngine(model, num_blocks=pages, block_size=page, max_batch=slots,
                                  use_hip_graphs=False, enable_prefix_caching=False, **kw)


def tokens_of(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def feed(engine, req, toks):
    """All positions' logits of one feed."""
    return engine.forward_batch([(req, toks)], [list(range(len(toks)))])


def assert_close(got, want, tol=2e-4):
    scale = want.abs().max().item()
    err = (got.cpu().float() - want).abs().max().item()
    assert err <= tol * max(scale, 1.0), f"max abs error {err} (scale {scale})"


def run_in_portions(engine, toks, cuts):
    """Feed toks in portions of the given sizes (the rest one by one); all logits."""
    req = engine.open_request()
    out, at = [], 0
    for c in cuts:
        c = min(c, len(toks) - at)
        if c <= 0:
            break
        out.append(feed(engine, req, toks[at:at + c]))
        at += c
    while at < len(toks):
        out.append(feed(engine, req, toks[at:at + 1]))
        at += 1
    engine.close_request(req)
    return torch.cat(out, dim=0)


SMALL = dict(heads=2, kv=1, dim=8, window=4, pool=2, rheads=1, rdim=7, mlp=False)
# a layer that uses another's weights repeats its entry
FULL = [layer(), layer(weights_of=0), layer(**SMALL), layer(**SMALL, weights_of=2), layer(weights_of=0)]


# -- each mechanism alone ------------------------------------------------------


@pytest.mark.parametrize("groups", [1, 2, 6])
def test_group_norm(groups):
    from megatron_amd.ops import ragged as R

    torch.manual_seed(0)
    x, y, w, w2 = torch.randn(7, 24), torch.randn(7, 24), torch.randn(24), torch.randn(24)
    xs = x.clone()
    a, b = R.residual_group_norm(xs, y, w, w2, groups, 1e-5, torch.float32)
    assert_close(a, O.group_rms_norm(x + y, w, groups, 1e-5), 1e-5)
    assert_close(b, O.group_rms_norm(x + y, w2, groups, 1e-5), 1e-5)
    assert_close(xs, x + y, 1e-6)


def _module_ctx(module, name, n, page, dtype=torch.float32, device="cpu"):
    pages = (n + page - 1) // page
    ctx = HybridInferenceContext(module.cache_spec(name, page), module.state_spec(name), pages + 2, page, 2,
                                 dtype=dtype, device=device)
    ctx.allocator.allocate(1)
    table = ctx.allocator.allocate(pages)[::-1]
    return ctx, table, ctx.acquire_slot()


@pytest.mark.parametrize("H,G,D,window,pool", [(4, 2, 6, 5, 3), (3, 3, 4, 1, 1), (2, 1, 8, 7, 4), (4, 4, 4, 64, 2),
                                               (2, 2, 4, 3, 9)])
def test_pooled_window_attention_alone(H, G, D, window, pool):
    from megatron_amd.transformer.pooled_window_attention import PooledWindowAttention

    torch.manual_seed(1)
    W, n, page = 16, 45, 8
    m = dict(heads=H, kv_heads=G, dim=D, vdim=D, scale=1.5, mask=dict(size=window, pool=pool))
    wt = {"q": torch.randn(H * D, W) / 4, "k": torch.randn(G * D, W) / 4, "o": torch.randn(W, H * D) / 4,
          "q.norm": 1 + 0.2 * torch.randn(H * D), "k.norm": 1 + 0.2 * torch.randn(G * D)}
    mod = PooledWindowAttention(W, H, G, D, D, 1.5, window, pool, 1e-5, dtype=torch.float32)
    with torch.no_grad():
        mod.w_in.copy_(torch.cat([wt["q"], wt["k"]]))
        mod.w_out.copy_(wt["o"])
        mod.q_norm.copy_(wt["q.norm"])
        mod.k_norm.copy_(wt["k.norm"])
    h = torch.randn(n, W)
    want = O.pooled_window_attention(h, wt, "", m, 1e-5)
    ctx, table, slot = _module_ctx(mod, "a", n, page)
    got, at = [], 0
    for c in (19, 2, 1, 13, 10):                      # portions: every block and window edge is cut somewhere
        ctx.begin_batch([c], [at], [slot], [table])
        with torch.no_grad():
            got.append(mod(h[at:at + c], ctx, "a"))
        at += c
    assert at == n
    assert_close(torch.cat(got), want, 1e-5)


@pytest.mark.parametrize("H,D,rank", [(2, 6, 3), (1, 10, 1), (3, 4, 5)])
def test_delta_rule_alone(H, D, rank):
    from megatron_amd.ssm.delta_rule import DeltaRuleMixer

    torch.manual_seed(2)
    W, n = 16, 33
    hd = H * D
    wt = {k: torch.randn(hd, W) / 4 for k in "rkvga"}
    wt.update({"w1": torch.randn(rank, W) / 4, "w2": torch.randn(hd, rank), "w0": torch.randn(hd) - 1,
               "a.b": torch.randn(hd), "norm": 1 + 0.2 * torch.randn(hd), "o": torch.randn(W, hd) / 4})
    mod = DeltaRuleMixer(W, H, D, rank, 1e-5, dtype=torch.float32)
    with torch.no_grad():
        mod.w_in.copy_(torch.cat([wt[k] for k in ("r", "k", "v", "g", "a", "w1")]))
        mod.w_out.copy_(wt["o"])
        mod.w2.copy_(wt["w2"]); mod.w0.copy_(wt["w0"]); mod.a_bias.copy_(wt["a.b"]); mod.norm_weight.copy_(wt["norm"])
    h = torch.randn(n, W)
    want = O.delta_rule(h, wt, "", dict(heads=H, dim=D), 1e-5)
    ctx, table, slot = _module_ctx(mod, "d", n, 8)
    got, at = [], 0
    for c in (17, 1, 2, 13):
        ctx.begin_batch([c], [at], [slot], [table])
        with torch.no_grad():
            got.append(mod(h[at:at + c], ctx, "d"))
        at += c
    assert_close(torch.cat(got), want, 1e-5)


def test_delta_rule_removes_along_the_key():
    """With full removal, no decay loss and a repeated key, the memory's answer
    for that key is replaced, not added to: a plain sum (no removal term) or a
    removal that read the updated state would answer differently."""
    from megatron_amd.ops import ragged_reference as ref

    D = 4
    k = torch.tensor([1.0, 2.0, -1.0, 0.5])
    v1, v2 = torch.tensor([1.0, 0, 0, 0]), torch.tensor([0, 3.0, 0, 0])
    big = 40.0
    # columns: r | k | v | g | a | w1(1)
    rows = []
    for v in (v1, v2):
        rows.append(torch.cat([k, k, v, torch.zeros(D), torch.full((D,), big), torch.zeros(1)]))
    proj = torch.stack(rows)
    state = torch.zeros(1, 1, D, D)

    class B:  # the one-request batch
        num_requests, host_cu, host_start, host_slots = 1, [0, 2], [0], [0]
    out = torch.zeros(2, D)
    ref.delta_rule_scan(proj, 0, D, 2 * D, 3 * D, 4 * D, 5 * D, 1, torch.zeros(D, 1), torch.full((D,), -big),
                        torch.zeros(D), torch.ones(D), 1, D, 0.0, state, B, out, 0, 1.0)
    S = state[0, 0]
    # after the second token the old association along u is gone: S^T k = |k|^2 v2 (+ nothing of v1)
    assert_close(S.T @ k, (k @ k) * v2, 1e-4)


@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (8, 1, 1, 1), (15, 4, 5, 3), (6, 3, 6, 4), (9, 3, 3, 3)])
def test_router_alone(E, top, groups, keep):
    from megatron_amd.ops import ragged as R

    torch.manual_seed(3)
    h, wr = torch.randn(50, 16), torch.randn(E, 16)
    rt = dict(experts=E, top=top, scale=1.3, groups=dict(count=groups, keep=keep))
    idx, wt = O.route(h, {"router": wr}, "", rt)
    ids, w = R.moe_route(h @ wr.T, E, top, groups, keep, 1.3)
    o1, o2 = idx.argsort(1), ids.long().argsort(1)
    assert torch.equal(idx.gather(1, o1), ids.long().gather(1, o2))
    assert_close(w.gather(1, o2), wt.gather(1, o1), 1e-6)


@pytest.mark.parametrize("shared", [None, 12])
def test_experts_alone(shared):
    cfg = make_config([layer(shared=shared)])
    w = make_weights(cfg, seed=4)
    blk = build(cfg, w).blocks["0"]
    torch.manual_seed(5)
    h = torch.randn(21, cfg["width"])
    with torch.no_grad():
        got = blk.mlp(h)
    assert_close(got, O.moe(h, w, "l0.mlp.", cfg["layers"][0]["mlp"]), 1e-5)


@pytest.mark.parametrize("kw", [dict(), dict(mlp=False), dict(groups=None, top=1), dict(kv=4), dict(kv=1, pool=1),
                                dict(window=1), dict(experts=4, groups=(4, 2), top=2, shared=None)],
                         ids=["default", "no-ff", "no-groups-top1", "mha", "mqa-pool1", "window1", "one-expert-groups"])
def test_single_layer_matches_oracle(kw):
    cfg = make_config([layer(**kw)])
    w = make_weights(cfg, seed=1)
    toks = tokens_of(37, cfg["vocab"], 2)
    got = build(cfg, w)(torch.tensor([toks]))[:, 0]
    assert_close(got, O.forward(cfg, w, toks))


# -- whole model through the engine -------------------------------------------------


def test_layers_and_shared_weights_match_oracle():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=6)
    toks = tokens_of(40, cfg["vocab"], 7)
    model = build(cfg, w)
    model.layer_trace = []
    eng = engine_for(model)
    req = eng.open_request()
    got = feed(eng, req, toks)
    trace = []
    want = O.forward(cfg, w, toks, trace)
    assert len(model.layer_trace) == len(trace) == len(FULL)
    for a, b in zip(model.layer_trace, trace):
        assert_close(a, b)
    assert_close(got, want)
    # layers that share weights keep caches and states of their own
    spec = model.inference_spec(8)
    assert {f"l{i}.left" for i in range(5)} <= set(spec.caches) and {f"l{i}.right.S" for i in range(5)} <= set(spec.states)
    assert len(list(model.blocks)) == 2


def test_prefill_then_decode_token_by_token():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=8)
    toks = tokens_of(48, cfg["vocab"], 9)
    want = O.forward(cfg, w, toks)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, [20]), want)          # 20 at once, then 28 single tokens
    assert_close(run_in_portions(eng, toks, []), want)            # everything token by token


@pytest.mark.parametrize("cuts", [[2, 2, 2, 3, 5, 2, 17, 2], [7, 1, 1, 9, 4, 4, 11], [31, 2], [3] * 16])
def test_portions(cuts):
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=10)
    toks = tokens_of(47, cfg["vocab"], 11)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, cuts), O.forward(cfg, w, toks))


def test_mixed_batch_equals_each_alone():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=12)
    V = cfg["vocab"]
    seqs = [tokens_of(n, V, 20 + i) for i, n in enumerate((45, 9, 30, 17))]
    want = [O.forward(cfg, w, s) for s in seqs]
    eng = engine_for(build(cfg, w), pages=60)
    reqs = [eng.open_request() for _ in seqs]
    at = [0] * 4
    got = [[] for _ in seqs]
    plan = [[(0, 13), (1, 2)], [(0, 1), (1, 1), (2, 11)], [(0, 20), (1, 1), (2, 1), (3, 17)],
            [(2, 18), (0, 1), (1, 5)], [(0, 10)]]
    for step in plan:
        feeds, wanted = [], []
        for i, n in step:
            feeds.append((reqs[i], seqs[i][at[i]:at[i] + n]))
            wanted.append(list(range(n)))
        out = eng.forward_batch(feeds, wanted)
        o = 0
        for i, n in step:
            got[i].append(out[o:o + n])
            at[i] += n
            o += n
    assert at == [len(s) for s in seqs]
    for g, wnt in zip(got, want):
        assert_close(torch.cat(g), wnt)


def test_freed_pages_and_slots_are_reused():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=13)
    V = cfg["vocab"]
    eng = engine_for(build(cfg, w), pages=9, slots=2)           # room for ~2 requests: everything is recycled
    for i, n in enumerate((33, 30, 35, 12, 36)):
        toks = tokens_of(n, V, 40 + i)
        assert_close(run_in_portions(eng, toks, [n // 2, 3]), O.forward(cfg, w, toks))
    assert eng.context.allocator.num_free == 9 and eng.context.slot_allocator.num_free == 2
    # two live at once, the second admitted into the slot and pages the first freed
    a, b, c = (tokens_of(n, V, 50 + n) for n in (30, 28, 31))
    ra, rb = eng.open_request(), eng.open_request()
    la = feed(eng, ra, a)
    lb1 = feed(eng, rb, b[:10])
    eng.close_request(ra)
    rc = eng.open_request()
    out = eng.forward_batch([(rb, b[10:]), (rc, c)], [list(range(18)), list(range(31))])
    assert_close(la, O.forward(cfg, w, a))
    assert_close(torch.cat([lb1, out[:18]]), O.forward(cfg, w, b))
    assert_close(out[18:], O.forward(cfg, w, c))


PEAK = dict(scale=6.0, window=9, pool=4, kv=2, heads=4, dim=6)     # peaked softmax: one key more or less shows


@pytest.mark.parametrize("n", list(range(8, 19)) + [33, 40, 41])
def test_window_and_block_edges_in_prompts_and_decoding(n):
    """Sequences whose last position puts the window's start and the newest
    visible block at every offset relative to block and page (8) borders."""
    cfg = make_config([layer(**PEAK), layer(**dict(PEAK, window=8, pool=8))])
    w = make_weights(cfg, seed=14, gain=1.5)
    toks = tokens_of(n, cfg["vocab"], 60 + n)
    want = O.forward(cfg, w, toks)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, [n]), want)            # prompt
    assert_close(run_in_portions(eng, toks, [n - 6]), want)        # the last six decoded one by one
    assert_close(run_in_portions(eng, toks, [5, n - 8, 2]), want)  # a portion that ends just before


def test_one_key_inside_or_outside_changes_the_answer():
    """The tests above can only fail if visibility matters: with the peaked
    configuration, moving the window edge by one changes the logits by far
    more than the comparison's tolerance."""
    base = make_config([layer(**PEAK)])
    other = make_config([layer(**dict(PEAK, window=PEAK["window"] + 1))])
    w = make_weights(base, seed=14, gain=1.5)
    toks = tokens_of(30, base["vocab"], 3)
    a, b = O.forward(base, w, toks), O.forward(other, w, toks)
    assert (a - b).abs().max() > 50 * 2e-4 * a.abs().max()
    pooled = make_config([layer(**dict(PEAK, pool=PEAK["pool"] + 1))])
    c = O.forward(pooled, w, toks)
    assert (a - c).abs().max() > 50 * 2e-4 * a.abs().max()


@pytest.mark.parametrize("P,first", [(4, 40), (3, 63), (5, 20)])      # blocks inside a page (8), across a page border
@pytest.mark.parametrize("decode", [False, True])
def test_far_key_is_seen_through_its_block(P, first, decode):
    """A key hundreds of tokens back that wins the softmax: its block's mean
    carries it.  The attention op on a designed cache: every key is small
    except one far block's, which is aligned with the last query; the query is
    part of the prompt, or decoded alone after it."""
    from megatron_amd.ops import ragged as R

    H = G = 1
    D, window, page, n = 8, 16, 8, 300
    rpp = (page + P - 1) // P
    ctx = HybridInferenceContext({"c": 2 * D, "c.pooled": (2 * D, rpp)}, {}, 40, page, 1, dtype=torch.float32, device="cpu")
    table = ctx.allocator.allocate((n + page - 1) // page)[::-1]
    torch.manual_seed(0)
    proj = torch.randn(n, 2 * D) * 0.05                             # [q | k], v = k
    direction = torch.zeros(D)
    direction[3] = 1.0
    assert first % P == 0 and first + P <= n - window
    proj[first:first + P, D:] += 3.0 * direction                    # one whole block
    proj[n - 1, :D] = 5.0 * direction
    ones = torch.ones(D)
    out = torch.zeros(n, D)
    for a, b in ([(0, n - 1), (n - 1, n)] if decode else [(0, n)]):
        ctx.begin_batch([b - a], [a], [0], [table])
        q = R.qk_norm_store(proj[a:b], 0, D, D, D, D, D, ones, ones, 1e-6, ctx.pools["c"], ctx.batch)
        R.pool_blocks(ctx.pools["c"], ctx.pools["c.pooled"], P, rpp, ctx.batch)
        R.pooled_window_attention(q, ctx.pools["c"], ctx.pools["c.pooled"], H, G, D, D, 4.0, window, P, rpp,
                                  ctx.batch, out[a:b], 0, 1.0)
    want_v = proj[first:first + P, D:].mean(0)
    assert_close(out[n - 1], want_v, 2e-2)                          # the far block dominates the answer
    # and the same query with the block's keys left small answers something else
    assert (out[n - 2] - want_v).abs().max() > 0.5


def test_first_tokens():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=15)
    for n in (1, 2, 3):
        toks = tokens_of(n, cfg["vocab"], 70 + n)
        eng = engine_for(build(cfg, w))
        assert_close(run_in_portions(eng, toks, [n]), O.forward(cfg, w, toks))
        assert_close(run_in_portions(eng, toks, []), O.forward(cfg, w, toks))


def test_long_decoding():
    cfg = make_config([layer(window=11, pool=5), layer(window=11, pool=5, weights_of=0)])
    w = make_weights(cfg, seed=16)
    toks = tokens_of(150, cfg["vocab"], 17)
    eng = engine_for(build(cfg, w), pages=24)
    assert_close(run_in_portions(eng, toks, [6]), O.forward(cfg, w, toks), 5e-4)


@pytest.mark.parametrize("kw,width,groups", [
    (dict(heads=6, kv=3, dim=4, rheads=3, rdim=4, experts=8, top=3, groups=(2, 1), ff=6, shared=5), 36, 1),
    (dict(heads=1, kv=1, dim=16, rheads=1, rdim=16, experts=2, top=2, groups=None, shared=None), 16, 16),
    (dict(heads=8, kv=2, dim=2, rheads=4, rdim=3, experts=5, top=5, groups=(1, 1), window=30, pool=30), 20, 5)])
def test_other_sizes(kw, width, groups):
    cfg = make_config([layer(**kw), layer(**kw), layer(**dict(kw, weights_of=1))], width=width, groups=groups, vocab=19)
    w = make_weights(cfg, seed=18, decay_rank=1 if width == 16 else 6)
    toks = tokens_of(70, cfg["vocab"], 19)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, [33, 2, 30]), O.forward(cfg, w, toks))


def test_greedy_generation_through_the_scheduler():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=20)
    V = cfg["vocab"]
    prompts = [tokens_of(n, V, 80 + n) for n in (19, 5, 26, 11, 8)]
    eng = engine_for(build(cfg, w), pages=30, slots=3, max_prefill_tokens=16)   # prompts are fed in portions
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=9, stop_on_eod=False))
    for p, r in zip(prompts, res):
        seq = list(p)
        for _ in range(9):
            lg = O.forward(cfg, w, seq)[-1]
            top2 = lg.topk(2).values
            assert top2[0] - top2[1] > 1e-3, "near-tie in the oracle: pick another seed"
            seq.append(int(lg.argmax()))
        assert r.output_tokens == seq[len(p):]
    assert eng.context.allocator.num_free == 30 and eng.context.slot_allocator.num_free == 3


def test_registry_builds_from_a_directory(tmp_path):
    import json

    from safetensors.torch import save_file

    from megatron_amd.models.registry import build_from_dir

    cfg = make_config(FULL)
    w = make_weights(cfg, seed=21)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    model = build_from_dir(str(tmp_path), dtype=torch.float32)
    toks = tokens_of(25, cfg["vocab"], 22)
    assert_close(model(torch.tensor([toks]))[:, 0], O.forward(cfg, w, toks))


# -- the same comparisons on the GPU kernels ---------------------------------------


# bf16 rounding may flip a close routing choice, which is no fault: the bf16 comparison
# uses layers whose experts are all chosen (weights stay continuous), with head sizes the
# matrix-core attention kernel takes
ALL_CHOSEN = dict(experts=3, top=3, groups=None)
BF16_FULL = [layer(dim=8, **ALL_CHOSEN), layer(dim=8, weights_of=0, **ALL_CHOSEN),
             layer(heads=6, kv=2, dim=16, window=12, pool=3, mlp=False)]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol,layers", [(torch.float32, 3e-4, FULL), (torch.float32, 3e-4, BF16_FULL),
                                              (torch.bfloat16, 6e-2, BF16_FULL)], ids=["fp32", "fp32-b", "bf16"])
def test_gpu_portions_and_mixed_batches(dtype, tol, layers):
    from megatron_amd.ops import ragged as R

    assert R._load("hybrid") is not None, "hybrid-ops extension must be built for GPU tests"
    cfg = make_config(layers)
    w = make_weights(cfg, seed=12)
    V = cfg["vocab"]
    eng = engine_for(build(cfg, w, dtype=dtype, device="cuda"), pages=60)
    toks = tokens_of(61, V, 30)
    want = O.forward(cfg, w, toks)
    assert_close(run_in_portions(eng, toks, [61]), want, tol)
    assert_close(run_in_portions(eng, toks, [2, 3, 17, 2, 30]), want, tol)
    seqs = [tokens_of(n, V, 31 + n) for n in (45, 9, 30)]
    reqs = [eng.open_request() for _ in seqs]
    o1 = eng.forward_batch([(reqs[0], seqs[0][:20]), (reqs[1], seqs[1][:8])], [list(range(20)), list(range(8))])
    o2 = eng.forward_batch([(reqs[0], seqs[0][20:]), (reqs[1], seqs[1][8:]), (reqs[2], seqs[2])],
                           [list(range(25)), [0], list(range(30))])
    assert_close(torch.cat([o1[:20], o2[:25]]), O.forward(cfg, w, seqs[0]), tol)
    assert_close(torch.cat([o1[20:], o2[25:26]]), O.forward(cfg, w, seqs[1]), tol)
    assert_close(o2[26:], O.forward(cfg, w, seqs[2]), tol)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [9, 13, 17, 40])
def test_gpu_window_and_block_edges(n):
    cfg = make_config([layer(**PEAK), layer(**dict(PEAK, window=8, pool=8))])
    w = make_weights(cfg, seed=14, gain=1.5)
    toks = tokens_of(n, cfg["vocab"], 60 + n)
    want = O.forward(cfg, w, toks)
    eng = engine_for(build(cfg, w, dtype=torch.float32, device="cuda"))
    assert_close(run_in_portions(eng, toks, [n]), want, 3e-4)
    assert_close(run_in_portions(eng, toks, [n - 6]), want, 3e-4)


@pytest.mark.gpu
def test_gpu_greedy_generation():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=20)
    V = cfg["vocab"]
    prompts = [tokens_of(n, V, 80 + n) for n in (19, 5, 26)]
    eng = engine_for(build(cfg, w, dtype=torch.float32, device="cuda"), pages=30, slots=3, max_prefill_tokens=16)
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, stop_on_eod=False))
    for p, r in zip(prompts, res):
        seq = list(p)
        for _ in range(6):
            seq.append(int(O.forward(cfg, w, seq)[-1].argmax()))
        assert r.output_tokens == seq[len(p):]


@pytest.mark.gpu
def test_gpu_grouped_and_looped_expert_paths_agree():
    """bf16 prompt portions run one grouped GEMM per linear over pairs sorted by expert
    (also with experts that get no pair); the per-expert loop must give the same rows."""
    from megatron_amd.moe.routed_experts import RoutedExpertsMLP

    torch.manual_seed(0)
    W, E, F_ = 64, 12, 40
    mlp = RoutedExpertsMLP(W, E, 2, F_, 1.25, groups=4, keep=1, route_scale=1.75, shared_ff=24, shared_limit=0.75)
    with torch.no_grad():
        for p in mlp.parameters():
            p.copy_(torch.randn(p.shape) * 0.2)
        mlp.w_router[[0, 5]] = -1.0          # with positive inputs these two never make a top 2 of 3
    mlp = mlp.cuda()
    h = torch.randn(50, W).abs().to(torch.bfloat16).cuda()
    add = torch.randn(50, W).to(torch.bfloat16).cuda()
    with torch.no_grad():
        a = mlp(h, add=add)
        os_env = __import__("os").environ
        os_env["MEGATRON_AMD_NO_TORCH_GROUPED"] = "1"
        try:
            b = mlp(h, add=add)
        finally:
            del os_env["MEGATRON_AMD_NO_TORCH_GROUPED"]
        ids, _, _ = mlp.route(h)
    assert len(set(ids.flatten().tolist())) < E, "the case is meant to leave experts without pairs"
    assert_close(a, b.cpu(), 2e-2)
