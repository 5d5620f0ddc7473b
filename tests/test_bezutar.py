"""Bezutar model family: the framework's ragged engine path against a plain
per-sequence oracle (tests/bezutar_oracle.py) on small random configurations.

Covers each mechanism alone, prefill against token-by-token decoding, prompt
portions down to two tokens, mixed batches against each request alone, reuse
of freed pages and state slots, salient keys far away / at page borders / at
the causal edge, the first tokens of a sequence, long decoding, optional
config sections and degenerate sizes, and greedy generation through the
engine's own scheduler.
"""

import copy
import math

import pytest
import torch

import bezutar_oracle as O
from megatron_amd.inference import DynamicInferenceEngine, SamplingParams
from megatron_amd.models.bezutar import BezutarConfig, BezutarModel, load_bezutar_state

ATT = dict(type="latent_attention",
           mixer=dict(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=20, q_rank=10, scale=0.31,
                      rot=dict(base=10000.0, dims=4, scaling=dict(factor=4.0, original=16, fast=4.0, slow=1.0))),
           mlp=dict(kind="dense", ff=24))
MLSTM = dict(type="mlstm", mixer=dict(heads=2, dim=6, vdim=10, gate_cap=7.0), mlp=dict(kind="dense", ff=24))
GRU = dict(type="mingru", mixer=dict(width=28), mlp=None)


def make_config(layers, width=16, vocab=37, streams=3, taps=3, bigram=True, max_positions=320, eps=1e-5):
    cfg = dict(architecture="Bezutar", vocab=vocab, width=width, max_positions=max_positions,
               norm=dict(eps=eps), layers=copy.deepcopy(layers))
    if streams:
        cfg["streams"] = streams
    if taps:
        cfg["canon"] = dict(taps=taps)
    if bigram:
        cfg["embedding"] = dict(bigram=dict(buckets=23, mul_prev=13, mul_cur=5))
    return cfg


def make_weights(cfg, seed=0, gain=1.0):
    """Random checkpoint tensors under the checkpoint's names (bf16-representable
    values so that both sides read the same numbers)."""
    g = torch.Generator().manual_seed(seed)
    W, out = cfg["width"], {}

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16).float()

    def lin(o, i):
        return rnd(o, i, scale=gain / math.sqrt(i))

    out["embed"] = rnd(cfg["vocab"], W)
    if cfg.get("embedding"):
        out["bigram"] = rnd(cfg["embedding"]["bigram"]["buckets"] + 1, W, scale=0.5)
    out["pos"] = rnd(cfg["max_positions"], W, scale=0.3)
    S = cfg.get("streams")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for q in (1, 2):
            if q == 2 and not L.get("mlp"):
                continue
            out[p + f"norm{q}"] = rnd(W, scale=0.2)
            if S:
                out[p + f"hc{q}.in"] = rnd(S, scale=0.6)
                out[p + f"hc{q}.out"] = rnd(S, scale=0.8)
                out[p + f"hc{q}.mix"] = (torch.eye(S) + rnd(S, S, scale=0.2)).to(torch.bfloat16).float()
        if cfg.get("canon"):
            out[p + "canon1"] = rnd(W, cfg["canon"]["taps"], scale=0.4)
        if L["type"] == "latent_attention":
            H, D, rd, vd, r, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out[p + "mix.dq"], out[p + "mix.dq.norm"] = lin(qr, W), 1 + rnd(qr, scale=0.1)
            out[p + "mix.uq"] = lin(H * (D + rd), qr)
            if m.get("kv_from") is None:
                out[p + "mix.dkv"], out[p + "mix.dkv.norm"] = lin(r + rd, W), 1 + rnd(r, scale=0.1)
            out[p + "mix.uk"], out[p + "mix.uv"] = lin(H * D, r), lin(H * vd, r)
            out[p + "mix.sink"], out[p + "mix.g"], out[p + "mix.o"] = rnd(H), lin(H, W), lin(W, H * vd)
        elif L["type"] == "mlstm":
            H, D, vd = m["heads"], m["dim"], m["vdim"]
            for n, rows in (("q", H * D), ("k", H * D), ("v", H * vd), ("g", H * vd), ("i", H), ("f", H)):
                out[p + "mix." + n] = lin(rows, W)
            out[p + "mix.i.b"], out[p + "mix.f.b"] = rnd(H), rnd(H) + 2
            out[p + "mix.norm"], out[p + "mix.o"] = 1 + rnd(H * vd, scale=0.1), lin(W, H * vd)
        else:
            C = m["width"]
            for n in "zxg":
                out[p + "mix." + n] = lin(C, W)
            out[p + "mix.z.b"], out[p + "mix.x.b"], out[p + "mix.o"] = rnd(C), rnd(C), lin(W, C)
        if L.get("mlp"):
            ff = L["mlp"]["ff"]
            out[p + "mlp.up"], out[p + "mlp.down"], out[p + "mlp.act"] = lin(ff, W), lin(W, ff), rnd(2)
    out["final.norm"], out["head"] = rnd(W, scale=0.2), lin(cfg["vocab"], W)
    return {k: v.to(torch.bfloat16).float() for k, v in out.items()}


def build(cfg, weights, dtype=torch.float32, device="cpu"):
    model = BezutarModel(BezutarConfig.from_dict(cfg, dtype=dtype))
    load_bezutar_state(model, weights)
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
    err = (got.cpu() - want).abs().max().item()
    assert err <= tol * max(scale, 1.0), f"max abs error {err} (scale {scale})"


FULL = [ATT, MLSTM, GRU, dict(ATT, mixer=dict(ATT["mixer"], kv_from=0)), MLSTM]


# -- each mechanism alone ------------------------------------------------------


@pytest.mark.parametrize("layer", [ATT, MLSTM, GRU], ids=["latent_attention", "mlstm", "mingru"])
@pytest.mark.parametrize("streams,taps", [(None, None), (3, 3)])
def test_single_mixer_matches_oracle(layer, streams, taps):
    cfg = make_config([dict(layer, mlp=None)], streams=streams, taps=taps, bigram=False)
    w = make_weights(cfg, seed=1)
    toks = tokens_of(29, cfg["vocab"], 2)
    got = build(cfg, w)(torch.tensor([toks]))[:, 0]
    assert_close(got, O.forward(w, cfg, toks))


def test_ops_against_oracle_functions():
    """Op level: the product's ragged ops against the oracle's per-mechanism
    functions on one sequence cut into two steps."""
    from megatron_amd.inference.contexts import HybridInferenceContext
    from megatron_amd.ops import ragged as R

    torch.manual_seed(3)
    T, W, taps = 21, 12, 4
    h = torch.randn(T, W)
    cw = torch.randn(W, taps)
    ctx = HybridInferenceContext({}, {"c": ((taps - 1, W), torch.float32), "g": ((W,), torch.float32)},
                                 8, 8, 2, dtype=torch.float32, device="cpu")
    slot, table = ctx.acquire_slot(), ctx.allocator.allocate(4)
    outs = []
    bz, bx = torch.randn(W), torch.randn(W)
    for a, b in ((0, 9), (9, T)):
        ctx.begin_batch([b - a], [a], [slot], [table])
        outs.append(R.canon_conv(h[a:b], cw, ctx.states["c"], ctx.batch, torch.float32))
    assert_close(torch.cat(outs), h + O.canon_conv(h, cw), 1e-5)
    Wd = {"p.z": torch.randn(W, W), "p.x": torch.randn(W, W), "p.g": torch.randn(W, W), "p.o": torch.eye(W),
          "p.z.b": bz, "p.x.b": bx}
    zxg2 = h @ torch.cat([Wd["p.z"], Wd["p.x"], Wd["p.g"]]).T
    ctx.states["g"].zero_()
    gru = []
    for a, b in ((0, 2), (2, 3), (3, T)):
        ctx.begin_batch([b - a], [a], [slot], [table])
        gru.append(R.mingru_scan(zxg2[a:b], bz, bx, ctx.states["g"], ctx.batch, torch.float32))
    assert_close(torch.cat(gru), O.mingru(Wd, "p.", dict(width=W), h, torch.float32), 1e-5)
    z0 = torch.linspace(-4, 4, 41)
    assert_close(R.xielu(z0, torch.tensor([0.4, -0.2]), torch.float32), O.xielu(z0, 0.4, -0.2), 1e-6)
    rot = dict(base=500.0, dims=8, scaling=dict(factor=3.0, original=24, fast=6.0, slow=1.5))
    cos, sin = R.rope_table(40, 8, 500.0, rot["scaling"])
    oc, os_ = O.yarn_tables(rot, 40, torch.float32)
    assert_close(cos, oc, 1e-6)
    assert_close(sin, os_, 1e-6)


# -- whole model ---------------------------------------------------------------


@pytest.fixture(scope="module")
def full():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=5)
    return cfg, w, build(cfg, w)


def test_layer_by_layer(full):
    cfg, w, model = full
    toks = tokens_of(19, cfg["vocab"], 6)
    want_layers = []
    want = O.forward(w, cfg, toks, layers_out=want_layers)
    model.layer_trace = []
    try:
        got = model(torch.tensor([toks]))[:, 0]
        for a, b in zip(model.layer_trace, want_layers):
            assert_close(a, b)
    finally:
        model.layer_trace = None
    assert_close(got, want)


def test_prefill_then_decode_token_by_token(full):
    cfg, w, model = full
    toks = tokens_of(70, cfg["vocab"], 7)
    want = O.forward(w, cfg, toks)
    eng = engine_for(model)
    req = eng.open_request()
    got = [feed(eng, req, toks[:33])] + [feed(eng, req, [t]) for t in toks[33:]]
    assert_close(torch.cat(got), want)
    eng.close_request(req)
    # and from the very first token on
    req = eng.open_request()
    got = torch.cat([feed(eng, req, [t]) for t in toks[:20]])
    assert_close(got, want[:20])


@pytest.mark.parametrize("sizes", [[2] * 20, [1, 2, 3, 5, 8, 13, 7, 1], [7, 2, 9, 2, 2, 16, 2], [37, 3]])
def test_portions(full, sizes):
    cfg, w, model = full
    toks = tokens_of(sum(sizes), cfg["vocab"], 8)
    want = O.forward(w, cfg, toks)
    eng = engine_for(model)
    req, got, at = eng.open_request(), [], 0
    for n in sizes:
        got.append(feed(eng, req, toks[at:at + n]))
        at += n
    assert_close(torch.cat(got), want)


def test_mixed_batch_equals_each_alone_and_reuses_pages_and_slots(full):
    cfg, w, model = full
    V = cfg["vocab"]
    seqs = {k: tokens_of(n, V, 10 + i) for i, (k, n) in enumerate(dict(a=41, b=9, c=26, d=3, e=30).items())}
    want = {k: O.forward(w, cfg, t) for k, t in seqs.items()}
    # pool too small for all five at once: e only fits once a and b have ended
    eng = engine_for(model, pages=14, page=8, slots=4)
    plan = [
        [("a", 17), ("b", 2)],
        [("a", 2), ("b", 1), ("c", 11)],
        [("a", 22), ("b", 6), ("c", 1), ("d", 3)],      # a, b, d end
        [("c", 1), ("e", 19)],
        [("e", 2), ("c", 13)],                          # c ends
        [("e", 9)],
    ]
    live, at, got = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    seen_slots, seen_pages = [], []
    for step in plan:
        feeds, names = [], []
        for k, n in step:
            if k not in live:
                live[k] = eng.open_request()
                seen_slots.append(live[k].slot)
            feeds.append((live[k], seqs[k][at[k]:at[k] + n]))
            names.append((k, n))
        out = eng.forward_batch(feeds, [list(range(n)) for _, n in names])
        row = 0
        for k, n in names:
            got[k].append(out[row:row + n])
            row += n
            at[k] += n
            if at[k] == len(seqs[k]):
                seen_pages += live[k].block_table
                eng.close_request(live.pop(k))
    assert len(seen_slots) > len(set(seen_slots)), "a state slot was used again"
    assert len(seen_pages) > len(set(seen_pages)), "pages were used again"
    for k in seqs:
        assert_close(torch.cat(got[k]), want[k])


def test_first_tokens(full):
    cfg, w, model = full
    for n in (1, 2, 3):
        toks = tokens_of(n, cfg["vocab"], 20 + n)
        assert_close(model(torch.tensor([toks]))[:, 0], O.forward(w, cfg, toks))


def test_long_decoding(full):
    cfg, w, model = full
    toks = tokens_of(230, cfg["vocab"], 30)
    want = O.forward(w, cfg, toks)
    eng = engine_for(model)
    req = eng.open_request()
    got = [feed(eng, req, toks[:5])] + [feed(eng, req, [t]) for t in toks[5:]]
    assert_close(torch.cat(got), want, 5e-4)


# -- other sizes and optional sections -----------------------------------------


@pytest.mark.parametrize("case", ["one_stream", "no_streams_no_canon_no_bigram", "taps2_head1", "partial_rot_no_yarn",
                                  "attention_last_shares_first", "wide"])
def test_other_configurations(case):
    a, m, g = copy.deepcopy(ATT), copy.deepcopy(MLSTM), copy.deepcopy(GRU)
    kw = {}
    if case == "one_stream":
        layers, kw = [a, g, m], dict(streams=1)
    elif case == "no_streams_no_canon_no_bigram":
        layers, kw = [m, a, g], dict(streams=None, taps=None, bigram=False)
    elif case == "taps2_head1":
        a["mixer"].update(heads=1, dim=4, vdim=12, kv_rank=9, q_rank=5)
        m["mixer"].update(heads=1, dim=5, vdim=3)
        layers, kw = [g, a, m], dict(taps=2, streams=2)
    elif case == "partial_rot_no_yarn":
        a["mixer"].update(rot_dim=8, rot=dict(base=77.0, dims=4))
        layers = [a, dict(a, mlp=None)]
    elif case == "attention_last_shares_first":
        a2 = copy.deepcopy(a)
        a2["mixer"]["kv_from"] = 0
        a2["mixer"].update(heads=2, dim=5, vdim=7, q_rank=6)      # own heads over the shared cache
        layers = [a, g, a2, a2]
    else:
        a["mixer"].update(heads=2, dim=16, rot_dim=16, vdim=24, kv_rank=72, q_rank=40,
                          rot=dict(base=1e5, dims=16, scaling=dict(factor=16.0, original=64, fast=16.0, slow=2.0)))
        m["mixer"].update(heads=2, dim=40, vdim=24)
        g["mixer"].update(width=100)
        layers, kw = [m, g, a], dict(width=48, vocab=90, streams=5, taps=5)
    cfg = make_config(layers, **kw)
    w = make_weights(cfg, seed=40)
    toks = tokens_of(45, cfg["vocab"], 41)
    want = O.forward(w, cfg, toks)
    eng = engine_for(build(cfg, w))
    req = eng.open_request()
    got = [feed(eng, req, toks[:11]), feed(eng, req, toks[11:13])] + [feed(eng, req, [t]) for t in toks[13:30]]
    got.append(feed(eng, req, toks[30:]))
    assert_close(torch.cat(got), want)


# -- keys that must (not) be seen --------------------------------------------


def _attention_probe(positions_of_marked, n_ctx, query_positions, page=8):
    """Pool rows are random except the marked positions, whose key part is a
    large multiple of the query direction: the output must be that row's latent
    when the marked key is visible (j <= query position) and must not contain
    it when it is not."""
    from megatron_amd.inference.contexts import HybridInferenceContext
    from megatron_amd.ops import ragged as R

    torch.manual_seed(11)
    H, rank, rd = 2, 12, 4
    Dk = rank + rd
    ctx = HybridInferenceContext({"kv": Dk}, {}, 64, page, 2, dtype=torch.float32, device="cpu")
    ctx.allocator.allocate(3)
    table = ctx.allocator.allocate((n_ctx + page - 1) // page)[::-1]
    slot = ctx.acquire_slot()
    direction = torch.randn(Dk)
    direction /= direction.norm()
    rows = torch.randn(n_ctx, Dk) * 0.1
    rows -= (rows @ direction)[:, None] * direction           # no accidental alignment
    for j in positions_of_marked:
        rows[j] = rows[j] + 40.0 * direction
    q0 = min(query_positions)
    ctx.begin_batch([n_ctx], [0], [slot], [table])
    ctx.pools["kv"][ctx.batch.tok_row] = rows
    n_q = len(query_positions)
    assert query_positions == list(range(q0, q0 + n_q))
    ctx.begin_batch([n_q], [q0], [slot], [table])
    q = direction.view(1, 1, Dk).expand(n_q, H, Dk).contiguous()
    out = R.latent_sink_attention(q, ctx.pools["kv"], rank, torch.zeros(H), 1.0, ctx.batch)
    return out, rows


@pytest.mark.parametrize("marked,n_ctx,queries", [
    (3, 300, [299]),            # far back, decoded alone
    (3, 300, list(range(280, 300))),   # far back, inside a prompt portion
    (7, 100, [99]), (8, 100, [99]),     # last row of a page / first row of the next
    (63, 100, list(range(60, 70))),     # marked key inside the portion: seen from its own place on
])
def test_salient_key_is_found_or_hidden(marked, n_ctx, queries):
    out, rows = _attention_probe([marked], n_ctx, queries)
    for i, p in enumerate(queries):
        for h in range(out.shape[1]):
            hit = (out[i, h] - rows[marked, :out.shape[2]]).abs().max().item()
            if p >= marked:
                assert hit < 1e-3, f"query at {p} lost the key at {marked}"
            else:
                # invisible: the output is a mix of the unmarked rows, all of which are small
                assert out[i, h].abs().max().item() < 1.0, f"query at {p} saw the future key at {marked}"


def test_sink_takes_its_share():
    """One visible key with score 0 and a sink logit s: the weight on the key is 1 / (1 + e^s)."""
    from megatron_amd.inference.contexts import HybridInferenceContext
    from megatron_amd.ops import ragged as R

    ctx = HybridInferenceContext({"kv": 6}, {}, 4, 4, 1, dtype=torch.float32, device="cpu")
    ctx.begin_batch([1], [0], [ctx.acquire_slot()], [ctx.allocator.allocate(1)])
    ctx.pools["kv"][ctx.batch.tok_row] = torch.tensor([[1.0, 2.0, 3.0, 4.0, 0.0, 0.0]])
    q = torch.zeros(1, 3, 6)
    sink = torch.tensor([0.0, 2.0, -30.0])
    out = R.latent_sink_attention(q, ctx.pools["kv"], 4, sink, 0.5, ctx.batch)
    for h in range(3):
        want = torch.tensor([1.0, 2.0, 3.0, 4.0]) / (1 + math.exp(float(sink[h])))
        assert_close(out[0, h], want, 1e-6)


def test_mlstm_remembers_far_token():
    """A value written once with a large input gate and kept by forget gates of ~1
    is read back many tokens later by a matching query, across steps."""
    from megatron_amd.inference.contexts import HybridInferenceContext
    from megatron_amd.ops import ragged as R

    H, D, V, T = 1, 4, 3, 200
    st = {"S": ((H, D, V), torch.float32), "n": ((H, D), torch.float32), "m": ((H,), torch.float32)}
    ctx = HybridInferenceContext({}, st, 4, 64, 1, dtype=torch.float32, device="cpu")
    slot, table = ctx.acquire_slot(), ctx.allocator.allocate(4)
    qkvg = torch.zeros(T, 2 * D + 2 * V)
    gates = torch.zeros(T, 2)
    gates[:, 0], gates[:, 1] = -20.0, 20.0            # write nothing, forget nothing
    key = torch.tensor([1.0, -1.0, 0.5, 2.0])
    qkvg[5, D:2 * D], qkvg[5, 2 * D:2 * D + V], gates[5, 0] = key, torch.tensor([3.0, -2.0, 1.0]), 5.0
    qkvg[-1, :D] = key
    qkvg[:, 2 * D + V:] = 30.0                         # output gate open
    outs = []
    for a, b in ((0, 100), (100, 199), (199, 200)):
        ctx.begin_batch([b - a], [a], [slot], [table])
        outs.append(R.mlstm_scan(qkvg[a:b], gates[a:b], torch.zeros(H), torch.zeros(H), torch.ones(V), H, D, V,
                                 50.0, 1e-6, ctx.states["S"], ctx.states["n"], ctx.states["m"], ctx.batch,
                                 torch.float32))
    o = outs[-1][0]
    want = torch.tensor([3.0, -2.0, 1.0])
    want = want / want.pow(2).mean().sqrt()
    assert_close(o, want, 1e-3)


# -- the engine's own entry point and scheduler ---------------------------------


def _oracle_greedy(w, cfg, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        t = int(O.forward(w, cfg, toks)[-1].argmax())
        out.append(t)
        toks.append(t)
    return out


def test_greedy_generation_through_scheduler(full):
    cfg, w, model = full
    V = cfg["vocab"]
    prompts = [tokens_of(n, V, 50 + n) for n in (13, 2, 27, 6, 1, 19)]
    # 4 slots, a small pool and an 11-token step budget: prompts are fed in
    # portions beside the running decodes, and later requests wait for slots
    eng = engine_for(model, pages=24, page=8, slots=4, max_prefill_tokens=11)
    res = eng.generate(prompts, SamplingParams(max_tokens=9, greedy=True, stop_on_eod=False))
    for p, r in zip(prompts, res):
        assert r.output_tokens == _oracle_greedy(w, cfg, p, 9)
    assert eng.context.allocator.num_free == 24 and eng.context.slot_allocator.num_free == 4


def test_bf16_serving_path_is_close(full):
    cfg, w, _ = full
    model = build(cfg, w, dtype=torch.bfloat16)
    toks = tokens_of(40, cfg["vocab"], 60)
    want = O.forward(w, cfg, toks)
    eng = engine_for(model)
    req = eng.open_request()
    got = torch.cat([feed(eng, req, toks[:25]), feed(eng, req, toks[25:])])
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    assert d.pow(2).mean().sqrt() < 0.08 * want.std()


def test_registry_builds_from_directory(tmp_path, full):
    import json

    from safetensors.torch import save_file

    from megatron_amd.models.registry import build_from_dir

    cfg, w, model = full
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()},
              str(tmp_path / "model.safetensors"))
    m2 = build_from_dir(str(tmp_path), dtype=torch.float32)
    toks = tokens_of(12, cfg["vocab"], 70)
    assert_close(m2(torch.tensor([toks])), model(torch.tensor([toks])), 1e-6)


# -- GPU: the HIP kernels in the same situations -------------------------------


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_engine_mixed_batch_against_oracle(dtype):
    from megatron_amd.ops import ragged as R

    assert R.has_native(), "ragged-ops extension must be built for GPU tests"
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=5)
    model = build(cfg, w, dtype=dtype, device="cuda")
    V = cfg["vocab"]
    seqs = {k: tokens_of(n, V, 80 + i) for i, (k, n) in enumerate(dict(a=90, b=17, c=33).items())}
    want = {k: O.forward(w, cfg, t) for k, t in seqs.items()}
    eng = engine_for(model, pages=20, page=8, slots=3)
    plan = [[("a", 40), ("b", 2)], [("a", 2), ("b", 1), ("c", 30)], [("a", 1), ("b", 14), ("c", 3)], [("a", 47)]]
    live, at, got = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in plan:
        feeds = []
        for k, n in step:
            live.setdefault(k, None)
            if live[k] is None:
                live[k] = eng.open_request()
            feeds.append((live[k], seqs[k][at[k]:at[k] + n]))
        out = eng.forward_batch(feeds, [list(range(n)) for _, n in step]).cpu()
        row = 0
        for k, n in step:
            got[k].append(out[row:row + n])
            row += n
            at[k] += n
    for k in seqs:
        g = torch.cat(got[k])
        if dtype == torch.float32:
            assert_close(g, want[k], 3e-4)
        else:
            d = g - want[k]
            d = d - d.mean(-1, keepdim=True)
            assert d.pow(2).mean().sqrt() < 0.08 * want[k].std()


@pytest.mark.gpu
def test_gpu_greedy_generation_matches_oracle():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=5)
    model = build(cfg, w, dtype=torch.float32, device="cuda")
    prompts = [tokens_of(n, cfg["vocab"], 50 + n) for n in (13, 2, 27, 6)]
    eng = engine_for(model, pages=24, page=8, slots=3, max_prefill_tokens=11)
    res = eng.generate(prompts, SamplingParams(max_tokens=7, greedy=True, stop_on_eod=False))
    for p, r in zip(prompts, res):
        assert r.output_tokens == _oracle_greedy(w, cfg, p, 7)
