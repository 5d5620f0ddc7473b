"""Context parallelism tests (reference analog: TE CP paths + core/utils
get_batch_on_this_cp_rank): ring attention and Ulysses a2a on gloo world 2
must match single-process full attention, forward and backward; end-to-end
tiny-GPT CP=2 loss matches CP=1."""

import torch

from megatron_amd.ops import reference as ref
from megatron_amd.parallel import grid as G
from megatron_amd.parallel.context_parallel import (
    cp_rope_positions,
    slice_for_cp_rank,
)
from tests.utils import assert_close, init_single, spawn_dist

S, B, HQ, HKV, D = 64, 2, 4, 2, 16


def _full_reference(seed=3):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(S, B, HQ, D, generator=g, requires_grad=True)
    k = torch.randn(S, B, HKV, D, generator=g, requires_grad=True)
    v = torch.randn(S, B, HKV, D, generator=g, requires_grad=True)
    dout = torch.randn(S, B, HQ, D, generator=g)
    out = ref.attention(q.float(), k.float(), v.float(), causal=True)
    out.backward(dout.float())
    return q, k, v, dout, out, q.grad, k.grad, v.grad


def _run_ring(rank, world):
    G.initialize_model_parallel(context_parallel_size=world)
    from megatron_amd.parallel.context_parallel import ring_attention

    q, k, v, dout, out_ref, dq_ref, dk_ref, dv_ref = _full_reference()
    qs = slice_for_cp_rank(q.detach(), rank, world, seq_dim=0).clone().requires_grad_(True)
    ks = slice_for_cp_rank(k.detach(), rank, world, seq_dim=0).clone().requires_grad_(True)
    vs = slice_for_cp_rank(v.detach(), rank, world, seq_dim=0).clone().requires_grad_(True)
    out = ring_attention(qs.float(), ks.float(), vs.float())
    out.backward(slice_for_cp_rank(dout, rank, world, seq_dim=0).float())
    assert_close(out, slice_for_cp_rank(out_ref, rank, world, seq_dim=0), rtol=1e-3, atol=1e-3)
    assert_close(qs.grad, slice_for_cp_rank(dq_ref, rank, world, seq_dim=0), rtol=1e-3, atol=1e-3)
    assert_close(ks.grad, slice_for_cp_rank(dk_ref, rank, world, seq_dim=0), rtol=1e-3, atol=1e-3)
    assert_close(vs.grad, slice_for_cp_rank(dv_ref, rank, world, seq_dim=0), rtol=1e-3, atol=1e-3)


def test_ring_attention_matches_full():
    spawn_dist(_run_ring, world_size=2)


def _run_ulysses(rank, world):
    G.initialize_model_parallel(context_parallel_size=world)
    from megatron_amd.parallel.context_parallel import ulysses_attention

    q, k, v, dout, out_ref, dq_ref, dk_ref, dv_ref = _full_reference()
    sl = lambda t: slice_for_cp_rank(t, rank, world, seq_dim=0, mode="a2a")
    qs = sl(q.detach()).clone().requires_grad_(True)
    ks = sl(k.detach()).clone().requires_grad_(True)
    vs = sl(v.detach()).clone().requires_grad_(True)
    out = ulysses_attention(qs.float(), ks.float(), vs.float())
    out.backward(sl(dout).float())
    assert_close(out, sl(out_ref), rtol=1e-3, atol=1e-3)
    assert_close(qs.grad, sl(dq_ref), rtol=1e-3, atol=1e-3)
    assert_close(ks.grad, sl(dk_ref), rtol=1e-3, atol=1e-3)
    assert_close(vs.grad, sl(dv_ref), rtol=1e-3, atol=1e-3)


def test_ulysses_attention_matches_full():
    spawn_dist(_run_ulysses, world_size=2)


def test_cp_rope_positions():
    pos = cp_rope_positions(64, 0, 2, "cpu")  # chunks 0 and 3
    assert pos.tolist() == list(range(0, 16)) + list(range(48, 64))
    pos = cp_rope_positions(64, 1, 2, "cpu")  # chunks 1 and 2
    assert pos.tolist() == list(range(16, 32)) + list(range(32, 48))
    pos = cp_rope_positions(64, 1, 2, "cpu", mode="a2a")
    assert pos.tolist() == list(range(32, 64))


def _loss_single(cfg_kwargs, tokens, labels):
    from megatron_amd.config import TransformerConfig
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel.random import model_parallel_seed

    init_single()
    model_parallel_seed(99)
    cfg = TransformerConfig(**cfg_kwargs)
    model = GPTModel(cfg)
    loss = model(tokens, labels=labels)  # [s, b]
    loss.sum().backward()
    g = model.decoder.layers[0].self_attention.linear_qkv.weight.grad.clone()
    G.destroy_model_parallel()
    return loss.detach(), g


def _run_gpt_cp(rank, world, cfg_kwargs, tokens, labels, loss_ref, grad_ref, mode):
    from megatron_amd.config import TransformerConfig
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel.random import model_parallel_seed

    G.initialize_model_parallel(context_parallel_size=world)
    model_parallel_seed(99)
    cfg = TransformerConfig(**{**cfg_kwargs, "context_parallel_size": world, "cp_comm_type": mode})
    model = GPTModel(cfg)
    t = slice_for_cp_rank(tokens, rank, world, seq_dim=1, mode=mode)
    l = slice_for_cp_rank(labels, rank, world, seq_dim=1, mode=mode)
    loss = model(t, labels=l)
    loss.sum().backward()
    ref_slice = slice_for_cp_rank(loss_ref.transpose(0, 1), rank, world, seq_dim=1, mode=mode)
    assert_close(loss.transpose(0, 1), ref_slice, rtol=2e-3, atol=2e-3)
    # grads of replicated weights: sum of CP shard grads == full grad
    g = model.decoder.layers[0].self_attention.linear_qkv.weight.grad.clone()
    import torch.distributed as dist

    dist.all_reduce(g)
    assert_close(g, grad_ref, rtol=5e-3, atol=5e-3)


def test_gpt_cp2_matches_single():
    cfg_kwargs = dict(num_layers=2, hidden_size=64, num_attention_heads=4,
                      num_query_groups=2, ffn_hidden_size=128, vocab_size=128,
                      max_position_embeddings=128)
    g = torch.Generator().manual_seed(11)
    tokens = torch.randint(0, 128, (2, 64), generator=g)
    labels = torch.randint(0, 128, (2, 64), generator=g)
    loss_ref, grad_ref = _loss_single(cfg_kwargs, tokens, labels)
    for mode in ("p2p", "a2a"):
        spawn_dist(_run_gpt_cp, 2, cfg_kwargs, tokens, labels, loss_ref, grad_ref, mode)


def test_balanced_cp_scheduler_assignments_complete():
    from megatron_amd.parallel.balanced_cp import BalancedCPScheduler

    sched = BalancedCPScheduler(world_size=8, max_cp=4, chunk_target=1024)
    seq_lens = [512, 1024, 4096, 2048, 8192, 256, 1024, 3072, 128, 6144]
    per_rank = sched.schedule(seq_lens)
    # every sample appears exactly once per member of its CP group, cp_ranks 0..cp-1
    seen = {}
    for r, assigns in per_rank.items():
        for a in assigns:
            seen.setdefault(a.sample, []).append((r, a.cp_rank, a.cp_size, a.ranks))
    assert set(seen.keys()) == set(range(len(seq_lens)))
    for i, entries in seen.items():
        cp = entries[0][2]
        assert len(entries) == cp
        ranks = sorted(e[0] for e in entries)
        assert tuple(ranks) == entries[0][3]
        assert ranks[0] % cp == 0  # aligned window
        assert sorted(e[1] for e in entries) == list(range(cp))


def test_balanced_cp_scheduler_balances_quadratic_work():
    import random

    from megatron_amd.parallel.balanced_cp import BalancedCPScheduler, quadratic_cost

    rng = random.Random(0)
    seq_lens = [rng.choice([256, 512, 1024, 2048, 4096, 8192]) for _ in range(64)]
    sched = BalancedCPScheduler(world_size=8, max_cp=8, chunk_target=1024)
    ratio = sched.balance_ratio(seq_lens)
    assert ratio < 1.15, ratio
    # naive fixed-CP=1 round-robin for comparison
    loads = [0.0] * 8
    for i, s in enumerate(seq_lens):
        loads[i % 8] += quadratic_cost(s)
    naive = max(loads) / (sum(loads) / 8)
    assert ratio <= naive


def test_pick_cp_size_powers_of_two():
    from megatron_amd.parallel.balanced_cp import pick_cp_size

    assert pick_cp_size(1024, 8, 4096) == 1
    assert pick_cp_size(8192, 8, 4096) == 2
    assert pick_cp_size(32768, 8, 4096) == 8
    assert pick_cp_size(10 ** 6, 4, 4096) == 4  # clamped at max_cp


def test_balanced_cp_fuzz():
    import random

    from megatron_amd.parallel.balanced_cp import BalancedCPScheduler

    for seed in range(5):
        rng = random.Random(seed)
        world = rng.choice([4, 8])
        sched = BalancedCPScheduler(world_size=world, max_cp=world,
                                    chunk_target=rng.choice([512, 2048]))
        seq_lens = [rng.randint(64, 16384) for _ in range(rng.randint(1, 40))]
        per_rank = sched.schedule(seq_lens)
        seen = {}
        for r, assigns in per_rank.items():
            for a in assigns:
                seen.setdefault(a.sample, set()).add(r)
        assert set(seen) == set(range(len(seq_lens)))
        for i, ranks in seen.items():
            assert len(ranks) == next(a.cp_size for aa in per_rank.values()
                                      for a in aa if a.sample == i)
        assert sched.balance_ratio(seq_lens) < 2.5


# --- hybrid (per-sample) CP wired through the scheduler ---------------------


def _hybrid_cp_case(rank, world):
    """Two samples of different lengths: the short one runs on ONE rank
    (cp=1), the long one ring-attends across both (cp=2); every output
    slice must equal the single-process full attention of its sample."""
    import torch.distributed as dist

    from megatron_amd.parallel import grid as G
    from megatron_amd.parallel.balanced_cp import BalancedCPScheduler
    from megatron_amd.parallel.context_parallel import cp_chunk_ids, slice_for_cp_rank
    from megatron_amd.parallel.hybrid_cp import (
        HybridCPGroups,
        build_hybrid_cp_batch,
        hybrid_cp_attention,
    )
    from megatron_amd.ops import reference as ref

    G.initialize_model_parallel()
    groups = HybridCPGroups(world)

    torch.manual_seed(7)
    b, h, d = 1, 2, 16
    lens = [8, 16]
    qkv = [tuple(torch.randn(L, b, h, d) for _ in range(3)) for L in lens]
    for tens in qkv:
        for t in tens:
            dist.broadcast(t, src=0)

    sched = BalancedCPScheduler(world_size=world, max_cp=world, chunk_target=8)
    per_rank = sched.schedule(lens)
    # slice q/k/v per assignment
    my = sorted(per_rank[rank], key=lambda a: a.sample)
    batch_qkv = []
    for a in my:
        q, k, v = qkv[a.sample]
        if a.cp_size == 1:
            batch_qkv.append((q, k, v))
        else:
            batch_qkv.append(tuple(
                slice_for_cp_rank(t, a.cp_rank, a.cp_size, seq_dim=0, mode="p2p")
                for t in (q, k, v)))
    outs = hybrid_cp_attention(batch_qkv, my, groups)

    for a, out in zip(my, outs):
        q, k, v = qkv[a.sample]
        full = ref.attention(q.float(), k.float(), v.float(), causal=True)
        if a.cp_size == 1:
            expect = full
        else:
            expect = slice_for_cp_rank(full, a.cp_rank, a.cp_size, seq_dim=0, mode="p2p")
        err = (out.float() - expect).abs().max()
        assert float(err) < 1e-4, (a, float(err))


def test_hybrid_cp_per_sample_groups():
    spawn_dist(_hybrid_cp_case, 2)


def test_build_hybrid_cp_batch_packs_slices():
    from megatron_amd.parallel.balanced_cp import BalancedCPScheduler
    from megatron_amd.parallel.hybrid_cp import build_hybrid_cp_batch

    sched = BalancedCPScheduler(world_size=2, max_cp=2, chunk_target=8)
    lens = [8, 16, 8]
    per_rank = sched.schedule(lens)
    samples = [torch.arange(L).float().unsqueeze(-1) for L in lens]
    total = 0
    for r in (0, 1):
        batch = build_hybrid_cp_batch(samples, per_rank, r)
        packed = batch.packed()
        assert packed.shape[0] == int(batch.cu_seqlens[-1])
        total += packed.shape[0]
    # every token placed exactly once across ranks
    assert total == sum(lens)


def _run_mla_cp(rank, world, cfg_kwargs, tokens, labels, loss_ref, grad_ref, mode):
    from megatron_amd.config import TransformerConfig
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel.random import model_parallel_seed

    G.initialize_model_parallel(context_parallel_size=world)
    model_parallel_seed(99)
    cfg = TransformerConfig(**{**cfg_kwargs, "context_parallel_size": world, "cp_comm_type": mode})
    model = GPTModel(cfg)
    t = slice_for_cp_rank(tokens, rank, world, seq_dim=1, mode=mode)
    l = slice_for_cp_rank(labels, rank, world, seq_dim=1, mode=mode)
    loss = model(t, labels=l)
    loss.sum().backward()
    ref_slice = slice_for_cp_rank(loss_ref.transpose(0, 1), rank, world, seq_dim=1, mode=mode)
    assert_close(loss.transpose(0, 1), ref_slice, rtol=2e-3, atol=2e-3)
    g = model.decoder.layers[0].self_attention.linear_kv_up.weight.grad.clone()
    import torch.distributed as dist

    dist.all_reduce(g)
    assert_close(g, grad_ref, rtol=5e-3, atol=5e-3)


def test_mla_cp2_matches_single():
    """MLA training under CP=2 (ring p2p AND ulysses a2a) matches CP=1:
    global RoPE positions + LSE-merged ring partials on the unequal
    dqk/dv head dims."""
    cfg_kwargs = dict(num_layers=2, hidden_size=64, num_attention_heads=4,
                      num_query_groups=4, ffn_hidden_size=128, vocab_size=128,
                      max_position_embeddings=128, multi_latent_attention=True,
                      q_lora_rank=48, kv_lora_rank=32, qk_nope_head_dim=16,
                      qk_rope_head_dim=16, v_head_dim=16)
    g = torch.Generator().manual_seed(13)
    tokens = torch.randint(0, 128, (2, 64), generator=g)
    labels = torch.randint(0, 128, (2, 64), generator=g)

    def grad_of(model):
        return model.decoder.layers[0].self_attention.linear_kv_up.weight.grad.clone()

    from megatron_amd.config import TransformerConfig
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel.random import model_parallel_seed

    init_single()
    model_parallel_seed(99)
    model = GPTModel(TransformerConfig(**cfg_kwargs))
    loss = model(tokens, labels=labels)
    loss.sum().backward()
    loss_ref, grad_ref = loss.detach(), grad_of(model)
    G.destroy_model_parallel()
    for mode in ("p2p", "a2a"):
        spawn_dist(_run_mla_cp, 2, cfg_kwargs, tokens, labels, loss_ref, grad_ref, mode)


def _run_gpt_cp_window(rank, world, cfg_kwargs, tokens, labels, loss_ref, grad_ref, mode):
    from megatron_amd.config import TransformerConfig
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel.random import model_parallel_seed

    G.initialize_model_parallel(context_parallel_size=world)
    model_parallel_seed(99)
    cfg = TransformerConfig(**{**cfg_kwargs, "context_parallel_size": world, "cp_comm_type": mode})
    model = GPTModel(cfg)
    t = slice_for_cp_rank(tokens, rank, world, seq_dim=1, mode=mode)
    l = slice_for_cp_rank(labels, rank, world, seq_dim=1, mode=mode)
    loss = model(t, labels=l)
    loss.sum().backward()
    ref_slice = slice_for_cp_rank(loss_ref.transpose(0, 1), rank, world, seq_dim=1, mode=mode)
    assert_close(loss.transpose(0, 1), ref_slice, rtol=2e-3, atol=2e-3)
    g = model.decoder.layers[0].self_attention.linear_qkv.weight.grad.clone()
    import torch.distributed as dist

    dist.all_reduce(g)
    assert_close(g, grad_ref, rtol=5e-3, atol=5e-3)


def test_gpt_cp2_sliding_window_matches_single():
    """Sliding-window attention under CP=2 (ring p2p with per-chunk-pair
    window masks, and Ulysses) equals the CP=1 windowed run — closes the
    'window not supported under CP' limitation."""
    cfg_kwargs = dict(num_layers=2, hidden_size=64, num_attention_heads=4,
                      num_query_groups=2, ffn_hidden_size=128, vocab_size=128,
                      max_position_embeddings=128, window_size=24)
    g = torch.Generator().manual_seed(17)
    tokens = torch.randint(0, 128, (2, 64), generator=g)
    labels = torch.randint(0, 128, (2, 64), generator=g)
    loss_ref, grad_ref = _loss_single(cfg_kwargs, tokens, labels)
    for mode in ("p2p", "a2a"):
        spawn_dist(_run_gpt_cp_window, 2, cfg_kwargs, tokens, labels, loss_ref,
                   grad_ref, mode)


def test_gpt_cp4_matches_single():
    """CP=4 ring (3 rotation hops, 8 zigzag chunks) and Ulysses at world 4
    equal the single run — the multi-hop path CP=2 never exercises."""
    cfg_kwargs = dict(num_layers=2, hidden_size=64, num_attention_heads=4,
                      num_query_groups=4, ffn_hidden_size=128, vocab_size=128,
                      max_position_embeddings=128)
    g = torch.Generator().manual_seed(23)
    tokens = torch.randint(0, 128, (2, 64), generator=g)
    labels = torch.randint(0, 128, (2, 64), generator=g)
    loss_ref, grad_ref = _loss_single(cfg_kwargs, tokens, labels)
    for mode in ("p2p", "a2a"):
        spawn_dist(_run_gpt_cp, 4, cfg_kwargs, tokens, labels, loss_ref, grad_ref, mode)
