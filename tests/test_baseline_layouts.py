"""BASELINE.json parallel layouts, shape-for-shape under gloo.

Each headline config's parallelism layout (TP=8; TP=4 x PP=2 interleaved;
EP=8 all-to-all) runs on a tiny model at its real world size (8 CPU ranks),
resharded from a single-process checkpoint, and must reproduce the
single-process first-step loss.  This is the gloo
matrix: every RCCL call pattern the 8-GPU bench will issue (TP AR/AG/RS,
PP p2p + interleaved schedule, EP a2a) exercised at the real group sizes.
"""

import json
import os

import pytest
import torch

from megatron_amd.checkpoint.checkpointing import load_checkpoint, save_checkpoint
from megatron_amd.config import DDPConfig, OptimizerConfig, TransformerConfig
from megatron_amd.models.gpt import GPTModel
from megatron_amd.parallel import grid as G
from megatron_amd.parallel.random import model_parallel_seed
from megatron_amd.training.training import setup_model_and_optimizer, train_step
from tests.utils import init_single, spawn_dist

SEQ = 16
VOCAB = 128


def _cfg(**kw):
    base = dict(
        num_layers=4, hidden_size=64, num_attention_heads=8, num_query_groups=8,
        vocab_size=VOCAB, ffn_hidden_size=128, gradient_accumulation_fusion=True,
    )
    base.update(kw)
    return TransformerConfig(**base)


def _provider(config, pre_process=True, post_process=True, vp_stage=None):
    torch.manual_seed(42)
    return GPTModel(config, pre_process=pre_process, post_process=post_process,
                    vp_stage=vp_stage)


def _gen_batches(n, mbs=2, seed=7):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(n):
        t = torch.randint(0, VOCAB, (mbs, SEQ + 1), generator=g)
        out.append({"tokens": t[:, :-1], "labels": t[:, 1:]})
    return out


def forward_step(data_iterator, model):
    batch = next(data_iterator)

    def loss_func(loss_sb):
        s = loss_sb.sum()
        return s, torch.tensor(loss_sb.numel()), {"loss_sum": s.detach()}

    return model(batch["tokens"], labels=batch["labels"]), loss_func


def _one_step(cfg, ckpt_dir, save=False):
    opt_cfg = OptimizerConfig(lr=1e-3, clip_grad=1.0)
    ddp_cfg = DDPConfig(grad_reduce_in_fp32=True, bucket_size=10_000)
    chunks, opt = setup_model_and_optimizer(_provider, cfg, opt_cfg, ddp_cfg)
    if save:
        save_checkpoint(ckpt_dir, chunks, opt, iteration=0)
    else:
        load_checkpoint(ckpt_dir, chunks, opt, load_rng=False)
    batches = _gen_batches(4)
    its = [iter(batches) for _ in chunks]
    return train_step(forward_step, its, chunks, opt, cfg, 4, SEQ, 2)


def _layout_case(rank, world, name, ckpt_dir):
    layouts = {
        "tp8": (dict(tensor_parallel_size=8), dict(tensor_parallel_size=8)),
        "tp4pp2": (dict(tensor_parallel_size=4, pipeline_parallel_size=2,
                        virtual_pipeline_parallel_size=2),
                   dict(tensor_parallel_size=4, pipeline_parallel_size=2,
                        virtual_pipeline_parallel_size=2, num_query_groups=4)),
        "ep8": (dict(expert_parallel_size=8),
                dict(expert_parallel_size=8, num_experts=8, moe_router_topk=2,
                     moe_ffn_hidden_size=32, moe_aux_loss_coeff=0.01)),
    }
    init_kw, cfg_kw = layouts[name]
    G.initialize_model_parallel(**init_kw)
    model_parallel_seed(1234)
    r = _one_step(_cfg(**cfg_kw), ckpt_dir)
    grid = G.get_grid()
    if (grid.is_pipeline_last_stage(ignore_virtual=True)
            and grid.rank_in("tp") == 0 and grid.rank_in("dp") == 0):
        with open(os.environ["LAYOUT_TEST_OUT"], "w") as f:
            json.dump([r["lm_loss"]], f)


def _single_ref(cfg_kw, ckpt_dir):
    init_single()
    model_parallel_seed(1234)
    return _one_step(_cfg(**cfg_kw), ckpt_dir, save=True)["lm_loss"]


@pytest.mark.parametrize("name,ref_kw", [
    ("tp8", {}),
    ("tp4pp2", dict(num_query_groups=4)),
    ("ep8", dict(num_experts=8, moe_router_topk=2, moe_ffn_hidden_size=32,
                 moe_aux_loss_coeff=0.01)),
])
def test_baseline_layout_matches_single(tmp_path, monkeypatch, name, ref_kw):
    out = tmp_path / f"{name}.json"
    ckpt = str(tmp_path / "ckpt")
    monkeypatch.setenv("LAYOUT_TEST_OUT", str(out))
    ref_loss = _single_ref(ref_kw, ckpt)
    spawn_dist(_layout_case, 8, name, ckpt)
    got = json.load(open(out))[0]
    assert abs(got - ref_loss) < 5e-4, (name, got, ref_loss)


def _tp2cp2_case(rank, world, ckpt_dir):
    from megatron_amd.parallel.context_parallel import slice_for_cp_rank

    G.initialize_model_parallel(tensor_parallel_size=2, context_parallel_size=2)
    model_parallel_seed(1234)
    cfg = _cfg(tensor_parallel_size=2, context_parallel_size=2)
    opt_cfg = OptimizerConfig(lr=1e-3, clip_grad=1.0)
    ddp_cfg = DDPConfig(grad_reduce_in_fp32=True, bucket_size=10_000)
    chunks, opt = setup_model_and_optimizer(_provider, cfg, opt_cfg, ddp_cfg)
    load_checkpoint(ckpt_dir, chunks, opt, load_rng=False)
    grid = G.get_grid()
    cp_rank = grid.rank_in("cp")

    def fwd(it, model):
        batch = next(it)
        t = slice_for_cp_rank(batch["tokens"], cp_rank, 2, seq_dim=1, mode="p2p")
        l = slice_for_cp_rank(batch["labels"], cp_rank, 2, seq_dim=1, mode="p2p")

        def loss_func(loss_sb):
            s = loss_sb.sum()
            return s, torch.tensor(loss_sb.numel()), {"loss_sum": s.detach()}

        return model(t, labels=l), loss_func

    batches = _gen_batches(4)
    r = train_step(fwd, [iter(batches)], chunks, opt, cfg, 4, SEQ, 2)
    if grid.rank_in("tp") == 0 and grid.rank_in("cp") == 0:
        with open(os.environ["LAYOUT_TEST_OUT"], "w") as f:
            json.dump([r["lm_loss"]], f)


def test_tp2_cp2_composition_matches_single(tmp_path, monkeypatch):
    """TP=2 x CP=2 (world 4): head-sharded ring attention over sequence
    shards, resharded from a single-process checkpoint, reproduces the
    single-process first-step loss."""
    out = tmp_path / "tc.json"
    ckpt = str(tmp_path / "ckpt")
    monkeypatch.setenv("LAYOUT_TEST_OUT", str(out))
    ref_loss = _single_ref({}, ckpt)
    spawn_dist(_tp2cp2_case, 4, ckpt)
    got = json.load(open(out))[0]
    assert abs(got - ref_loss) < 2e-3, (got, ref_loss)


def _dp8_case(rank, world, ckpt_dir):
    """DP=8 (the Llama-3-8B headline layout): per-rank data shards, dist-opt
    ZeRO-1, loss equals the single-process run over the union batch."""
    G.initialize_model_parallel()
    model_parallel_seed(1234)
    cfg = _cfg()
    opt_cfg = OptimizerConfig(lr=1e-3, clip_grad=1.0, use_distributed_optimizer=True)
    ddp_cfg = DDPConfig(grad_reduce_in_fp32=True, bucket_size=10_000,
                        use_distributed_optimizer=True)
    chunks, opt = setup_model_and_optimizer(_provider, cfg, opt_cfg, ddp_cfg)
    load_checkpoint(ckpt_dir, chunks, opt, load_rng=False)
    batches = _gen_batches(8)
    mine = [batches[rank]]
    r = train_step(forward_step, [iter(mine)], chunks, opt, cfg, 1, SEQ, 2)
    if rank == 0:
        with open(os.environ["LAYOUT_TEST_OUT"], "w") as f:
            json.dump([r["lm_loss"]], f)


def test_dp8_matches_single(tmp_path, monkeypatch):
    out = tmp_path / "dp8.json"
    ckpt = str(tmp_path / "ckpt")
    monkeypatch.setenv("LAYOUT_TEST_OUT", str(out))
    init_single()
    model_parallel_seed(1234)
    cfg = _cfg()
    opt_cfg = OptimizerConfig(lr=1e-3, clip_grad=1.0, use_distributed_optimizer=True)
    ddp_cfg = DDPConfig(grad_reduce_in_fp32=True, bucket_size=10_000,
                        use_distributed_optimizer=True)
    chunks, opt = setup_model_and_optimizer(_provider, cfg, opt_cfg, ddp_cfg)
    save_checkpoint(ckpt, chunks, opt, iteration=0)
    r = train_step(forward_step, [iter(_gen_batches(8))], chunks, opt, cfg, 8, SEQ, 2)
    ref_loss = r["lm_loss"]
    spawn_dist(_dp8_case, 8, ckpt)
    got = json.load(open(out))[0]
    assert abs(got - ref_loss) < 5e-4, (got, ref_loss)
