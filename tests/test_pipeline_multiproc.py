"""Multi-process pipeline tests over gloo on localhost (world_size=2) —
the CPU analog of the reference's loopback-TCP multi-node integration tests
(reference tests/conftest.py:18-22 runs real User/Worker/Validator processes
on 127.0.0.1; here real ranks run the real SPMD pipeline over gloo)."""

import os
import sys

import pytest
import torch
import torch.multiprocessing as mp

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _port(offset: int) -> int:
    """Distinct, pid-varying rendezvous ports (avoids TIME_WAIT rebind
    flakes when suites re-run quickly)."""
    return 20000 + (os.getpid() * 13 + offset * 101) % 20000


def _gen_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.planner import plan_for_world
    from tensorlink_amd.parallel.pipeline import PipelineRunner, SamplingParams
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", world)
    r = PipelineRunner(plan, rank, world, device=torch.device("cpu"))
    torch.manual_seed(7)
    ids = torch.randint(0, 1024, (4, 12)) if rank == 0 else None
    out = r.generate(ids, SamplingParams(max_new_tokens=6))
    if rank == 0:
        q.put(out)
    dist.destroy_process_group()


def _train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.planner import plan_for_world
    from tensorlink_amd.parallel.pipeline import PipelineTrainer
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", world, training=True)
    tr = PipelineTrainer(plan, rank, world, device=torch.device("cpu"),
                         lr=1e-3)
    torch.manual_seed(3)
    ids = torch.randint(0, 1024, (8, 16)) if rank == 0 else None
    losses = [tr.train_step(ids, ids, n_micro=4) for _ in range(4)]
    if rank == 0:
        q.put(losses)
    dist.destroy_process_group()


def _run(worker, world, port, timeout=240, retries=2):
    last_exc = None
    for attempt in range(retries + 1):
        ctx = mp.get_context("spawn")
        q = ctx.Queue()
        ps = [ctx.Process(target=worker,
                          args=(r, world, port + attempt * 7, q))
              for r in range(world)]
        for p in ps:
            p.start()
        try:
            result = q.get(timeout=timeout)
            return result
        except Exception as e:   # transient spawn/rendezvous flake: retry
            last_exc = e
        finally:
            for p in ps:
                p.join(30)
                if p.is_alive():
                    p.terminate()
    raise last_exc


def _run_collect(worker, world, port, n_results=None, timeout=240,
                 retries=2):
    """Like _run but collects one result per expected sender, with the
    same transient-flake retry."""
    n_results = world if n_results is None else n_results
    last_exc = None
    for attempt in range(retries + 1):
        ctx = mp.get_context("spawn")
        q = ctx.Queue()
        ps = [ctx.Process(target=worker,
                          args=(r, world, port + attempt * 7, q))
              for r in range(world)]
        for p in ps:
            p.start()
        try:
            results = [q.get(timeout=timeout) for _ in range(n_results)]
            return results
        except Exception as e:
            last_exc = e
        finally:
            for p in ps:
                p.join(30)
                if p.is_alive():
                    p.terminate()
    raise last_exc


@pytest.mark.timeout(300)
def test_pp2_generate_matches_reference():
    out = _run(_gen_worker, 2, _port(1))
    assert out.shape == (4, 6)

    # single-process reference with identical per-stage seeds
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 2)
    stages = []
    for rk in range(2):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=rk)
        stages.append(st)
    torch.manual_seed(7)
    ids = torch.randint(0, 1024, (4, 12))
    cur = ids
    for _ in range(6):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(4, -1).contiguous()
        h = stages[0](cur, pos, return_logits=False)
        logits = stages[1](h, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert torch.equal(cur[:, 12:], out)


@pytest.mark.timeout(300)
def test_pp2_1f1b_training_reduces_loss():
    losses = _run(_train_worker, 2, _port(2))
    assert len(losses) == 4
    assert losses[-1] < losses[0]


def _dp_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.dp import HybridTrainer
    init_distributed(backend="gloo")
    tr = HybridTrainer("tiny", rank, world, dp=2, device=torch.device("cpu"),
                       lr=1e-3)
    torch.manual_seed(5)
    ids = torch.randint(0, 1024, (8, 16)) if rank == 0 else None
    losses = [tr.train_step(ids, ids, n_micro=2) for _ in range(4)]
    # replicas must remain bit-identical after synced steps
    h = float(tr.optimizer.flat_param.double().sum())
    q.put((rank, losses, h))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_dp2_training_replicas_stay_synced():
    results = {rank: (losses, h) for rank, losses, h in
               _run_collect(_dp_worker, 2, _port(3))}
    l0, h0 = results[0]
    l1, h1 = results[1]
    assert l0 == l1, "losses must agree across replicas"
    assert l0[-1] < l0[0]
    assert abs(h0 - h1) < 1e-6, "replica weights diverged"


def _engine_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.engine.engine import InferenceEngine
    from tensorlink_amd.parallel.comm import init_distributed
    init_distributed(backend="gloo")
    eng = InferenceEngine(rank=rank, world=world,
                          device=torch.device("cpu"))
    if rank != 0:
        eng.worker_loop()
        return
    eng.load_model("tiny")
    resp = eng.generate({"hf_name": "tiny", "message": "hello",
                         "max_new_tokens": 6, "do_sample": False,
                         "output_format": "simple"})
    chunks = list(eng.generate_stream({
        "hf_name": "tiny", "message": "hi", "max_new_tokens": 4,
        "do_sample": False, "output_format": "simple"}))
    eng.shutdown()
    q.put((resp, chunks))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_engine_serving_over_pp2():
    """Full serving stack (engine + worker_loop) across 2 pipeline ranks —
    the reference's validator+worker serving topology on gloo loopback."""
    resp, chunks = _run_collect(_engine_worker, 2, _port(4),
                                n_results=1)[0]
    assert "response" in resp and resp["model"] == "tiny"
    assert chunks[-1] == "data: [DONE]\n\n"
    assert len(chunks) >= 2


def _gen4_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.planner import plan_for_world
    from tensorlink_amd.parallel.pipeline import PipelineRunner, SamplingParams
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", world)
    r = PipelineRunner(plan, rank, world, device=torch.device("cpu"))
    torch.manual_seed(21)
    ids = torch.randint(0, 1024, (8, 12)) if rank == 0 else None
    out = r.generate(ids, SamplingParams(max_new_tokens=5))
    if rank == 0:
        q.put(out)
    dist.destroy_process_group()


@pytest.mark.timeout(420)
def test_pp4_ring_decode_matches_reference():
    """4-stage ring-pipelined decode (the SCALE-bench shape) vs a
    single-process stage-chained reference."""
    out = _run(_gen4_worker, 4, _port(5), timeout=360)
    assert out.shape == (8, 5)
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 4)
    stages = []
    for rk in range(4):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=rk)
        stages.append(st)
    torch.manual_seed(21)
    ids = torch.randint(0, 1024, (8, 12))
    cur = ids
    for _ in range(5):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(8, -1).contiguous()
        h = cur
        for st in stages[:-1]:
            h = st(h, pos, return_logits=False)
        logits = stages[-1](h, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert torch.equal(cur[:, 12:], out)


def _tp_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.pipeline import SamplingParams
    from tensorlink_amd.parallel.tp import TPRunner
    init_distributed(backend="gloo")
    r = TPRunner("tiny", rank, world, device=torch.device("cpu"), seed=7)
    torch.manual_seed(31)
    ids = torch.randint(0, 1024, (3, 14))
    out = r.generate(ids, SamplingParams(max_new_tokens=6))
    q.put((rank, out))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_tp2_matches_single_rank_reference():
    """Tensor parallelism: 2 head-sharded ranks with per-layer all-reduce
    reproduce the single-rank greedy output."""
    outs = dict(_run_collect(_tp_worker, 2, _port(6)))
    # both ranks computed the same tokens (logits agree post all-reduce)
    assert torch.equal(outs[0], outs[1])

    # single-rank reference from the same seeded full init
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.models.configs import get_config
    m = build_full_model(get_config("tiny"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=7)
    torch.manual_seed(31)
    ids = torch.randint(0, 1024, (3, 14))
    cur = ids
    for _ in range(6):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(3, -1).contiguous()
        logits = m(cur, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert torch.equal(cur[:, 14:], outs[0])


def _train4_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.planner import plan_for_world
    from tensorlink_amd.parallel.pipeline import PipelineTrainer
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", world, training=True)
    tr = PipelineTrainer(plan, rank, world, device=torch.device("cpu"),
                         lr=1e-3)
    torch.manual_seed(13)
    ids = torch.randint(0, 1024, (8, 16)) if rank == 0 else None
    losses = [tr.train_step(ids, ids, n_micro=8) for _ in range(3)]
    if rank == 0:
        q.put(losses)
    dist.destroy_process_group()


@pytest.mark.timeout(420)
def test_pp4_1f1b_training(port_offset=7):
    """BASELINE config #3 shape: 1F1B training across 4 pipeline stages."""
    losses = _run(_train4_worker, 4, _port(7), timeout=360)
    assert losses[-1] < losses[0], losses


def _ep_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.ep import EPRunner
    from tensorlink_amd.parallel.pipeline import SamplingParams
    init_distributed(backend="gloo")
    r = EPRunner("tiny-moe", rank, world, device=torch.device("cpu"), seed=9)
    torch.manual_seed(41)
    ids = torch.randint(0, 1024, (2, 10))
    out = r.generate(ids, SamplingParams(max_new_tokens=5))
    q.put((rank, out))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_ep2_matches_single_rank_reference():
    """Expert parallelism: 2 ranks each holding half the experts (partial
    sums all-reduced) reproduce the single-rank MoE output."""
    outs = dict(_run_collect(_ep_worker, 2, _port(8)))
    assert torch.equal(outs[0], outs[1])

    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.models.configs import get_config
    m = build_full_model(get_config("tiny-moe"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=9)
    torch.manual_seed(41)
    ids = torch.randint(0, 1024, (2, 10))
    cur = ids
    for _ in range(5):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(2, -1).contiguous()
        logits = m(cur, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert torch.equal(cur[:, 10:], outs[0])


def _cp_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.cp import CPRunner
    init_distributed(backend="gloo")
    r = CPRunner("tiny", rank, world, device=torch.device("cpu"), seed=17)
    torch.manual_seed(51)
    ids = torch.randint(0, 1024, (2, 24))
    logits = r.forward_logits(ids)
    q.put((rank, logits))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_cp2_ring_attention_matches_single_rank():
    """Context parallelism: 2 sequence-sharded ranks with ring attention
    reproduce single-rank prefill logits."""
    outs = dict(_run_collect(_cp_worker, 2, _port(9)))
    cp_logits = torch.cat([outs[0], outs[1]], dim=1)     # [B, S, V]

    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.models.configs import get_config
    m = build_full_model(get_config("tiny"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=17)
    torch.manual_seed(51)
    ids = torch.randint(0, 1024, (2, 24))
    pos = torch.arange(24).unsqueeze(0).expand(2, -1).contiguous()
    ref = m(ids, pos)
    torch.testing.assert_close(cp_logits, ref, atol=1e-4, rtol=1e-4)


def _tp_train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.tp import TPTrainer
    init_distributed(backend="gloo")
    tr = TPTrainer("tiny", rank, world, device=torch.device("cpu"), seed=9,
                   lr=1e-3)
    torch.manual_seed(41)
    batches = [torch.randint(0, 1024, (2, 24)) for _ in range(3)]
    losses = [tr.train_step(b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_tp2_training_matches_single_rank():
    """TP training (differentiable f/g collectives): 2 sharded ranks
    reproduce the single-rank loss trajectory over 3 optimizer steps."""
    outs = dict(_run_collect(_tp_train_worker, 2, _port(11)))
    assert outs[0] == pytest.approx(outs[1], rel=1e-4)

    import torch
    from tensorlink_amd import ops as tl_ops
    from tensorlink_amd.models.configs import get_config
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.optim import FusedAdamW
    m = build_full_model(get_config("tiny"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=9)
    m.train()
    for p in m.parameters():
        p.requires_grad_(True)
    opt = FusedAdamW(m.parameters(), lr=1e-3, weight_decay=0.01)
    torch.manual_seed(41)
    batches = [torch.randint(0, 1024, (2, 24)) for _ in range(3)]
    ref_losses = []
    for ids in batches:
        B, S = ids.shape
        pos = torch.arange(S, dtype=torch.int32
                           ).unsqueeze(0).expand(B, -1).contiguous()
        opt.zero_grad()
        logits = m.head(m(ids, pos, training=True, return_logits=False))
        loss = tl_ops.causal_lm_loss(logits, ids)
        loss.backward()
        opt.step()
        ref_losses.append(float(loss.detach()))
    assert outs[0] == pytest.approx(ref_losses, rel=2e-3)


def _ep_a2a_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.ep import EPRunner
    from tensorlink_amd.parallel.pipeline import SamplingParams
    init_distributed(backend="gloo")
    r = EPRunner("tiny-moe", rank, world, device=torch.device("cpu"),
                 seed=9, mode="alltoall")
    torch.manual_seed(41)
    ids = torch.randint(0, 1024, (2, 10))
    out = r.generate(ids, SamplingParams(max_new_tokens=5))
    q.put((rank, out))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_ep2_alltoall_matches_single_rank():
    """Token-routing EP: tokens sharded, dispatched to expert-owner ranks
    with uneven all_to_all, combined and all-gathered — reproduces the
    single-rank MoE output exactly (incl. S=1 decode where some ranks
    get an empty token shard)."""
    outs = dict(_run_collect(_ep_a2a_worker, 2, _port(13)))
    assert torch.equal(outs[0], outs[1])

    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.models.configs import get_config
    m = build_full_model(get_config("tiny-moe"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=9)
    torch.manual_seed(41)
    ids = torch.randint(0, 1024, (2, 10))
    cur = ids
    for _ in range(5):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(2, -1).contiguous()
        logits = m(cur, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert torch.equal(cur[:, 10:], outs[0])


def _cp_gen_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.cp import CPRunner
    init_distributed(backend="gloo")
    r = CPRunner("tiny", rank, world, device=torch.device("cpu"), seed=17)
    torch.manual_seed(53)
    ids = torch.randint(0, 1024, (2, 24))
    out = r.generate(ids, max_new_tokens=6)
    q.put((rank, out))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_cp2_decode_matches_single_rank():
    """CP decode: sequence-sharded KV cache (prompt chunks stay on their
    prefill rank, decode tokens append to the last rank) with per-step
    (o,m,l) all-gather merge reproduces single-rank greedy decode."""
    outs = dict(_run_collect(_cp_gen_worker, 2, _port(15)))
    assert torch.equal(outs[0], outs[1])

    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.models.configs import get_config
    m = build_full_model(get_config("tiny"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=17)
    torch.manual_seed(53)
    ids = torch.randint(0, 1024, (2, 24))
    cur = ids
    for _ in range(6):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(2, -1).contiguous()
        logits = m(cur, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert torch.equal(cur[:, 24:], outs[0])


def _elastic_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import time
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.elastic import ElasticRunner
    from tensorlink_amd.parallel.pipeline import SamplingParams
    init_distributed(backend="gloo")
    ckpt = os.environ["TL_ELASTIC_CKPT"]
    r = ElasticRunner("tiny", device=torch.device("cpu"), seed=23,
                      rendezvous_port=port + 100, grace_s=1.0)
    r.save_checkpoint(ckpt)              # both stage shards on disk
    dist.barrier()
    torch.manual_seed(61)
    ids = torch.randint(0, 1024, (1, 12))
    out1 = r.generate(ids, SamplingParams(max_new_tokens=4))
    if rank == 1:
        os._exit(0)                      # simulated crash: no teardown
    time.sleep(2.0)                      # let rank 1 die first
    out2 = r.generate(ids, SamplingParams(max_new_tokens=4))
    # plain lists: the worker exits right after put, so shared-memory
    # tensor handles would race the parent's fd dup
    q.put((rank, (out1.tolist(), out2.tolist(), r.world, r.generation)))


@pytest.mark.timeout(300)
def test_elastic_recovery_after_rank_loss(tmp_path):
    """Rank 1 dies mid-service: rank 0's next collective fails, survivors
    re-rendezvous on a side store, the group re-forms as world=1, the
    pipeline is re-planned and reloaded from the per-stage checkpoint
    (re-partitioned pp2 -> pp1), and the retried request reproduces the
    pre-failure output."""
    os.environ["TL_ELASTIC_CKPT"] = str(tmp_path / "ckpt")
    try:
        outs = dict(_run_collect(_elastic_worker, 2, _port(17),
                                 n_results=1))
    finally:
        del os.environ["TL_ELASTIC_CKPT"]
    out1, out2, new_world, gen = outs[0]
    assert new_world == 1 and gen == 1
    assert out1 == out2                  # same weights, same tokens


def _pp_batch_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.engine.engine import InferenceEngine
    from tensorlink_amd.parallel.comm import init_distributed
    init_distributed(backend="gloo")
    eng = InferenceEngine(rank=rank, world=world, device=torch.device("cpu"))
    if rank != 0:
        eng.worker_loop()
        return
    eng.load_model("tiny", continuous=True, max_slots=5, max_ctx=256,
                   prefill_chunk=16)
    b = eng.jobs["tiny"].batcher
    torch.manual_seed(33)
    # 5 concurrent slots > world: exercises multi-group pipelined decode
    prompts = [torch.randint(0, 1024, (n,)) for n in (30, 9, 21, 40, 5)]
    reqs = [b.submit(p, max_new_tokens=8) for p in prompts]
    outs = [rq.result(timeout=120) for rq in reqs]
    # releases are deferred one scheduler iteration (rank sync) — wait
    import time
    for _ in range(200):
        if b.cache.allocator.n_free == b.cache.allocator.n_pages:
            break
        time.sleep(0.02)
    n_free = b.cache.allocator.n_free
    n_pages = b.cache.allocator.n_pages
    eng.unload_model("tiny")
    eng.shutdown()
    q.put((rank, ([p.tolist() for p in prompts], outs, n_free, n_pages,
                  b.steps)))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_pp2_continuous_batching_matches_serial():
    """PP-aware continuous batching: rank 0 schedules, followers execute
    stage commands; concurrent chunked-prefill requests across a 2-stage
    pipeline reproduce single-rank serial greedy outputs and all pages
    return to the pool."""
    outs = dict(_run_collect(_pp_batch_worker, 2, _port(19), n_results=1))
    prompts, results, n_free, n_pages, steps = outs[0]
    assert n_free == n_pages, "pages leaked"
    assert steps < 3 * 8          # interleaved, not serial

    import torch
    from tensorlink_amd.parallel.pipeline import PipelineRunner, SamplingParams
    from tensorlink_amd.parallel.planner import plan_for_world
    # single-rank reference with the same per-stage seeds as the pp2 pair
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    plan = plan_for_world("tiny", 2)
    stages = []
    for rk in range(2):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=rk)
        stages.append(st)
    for p, o in zip(prompts, results):
        cur = torch.tensor(p, dtype=torch.int64).unsqueeze(0)
        toks = []
        for _ in range(8):
            pos = torch.arange(cur.shape[1]).unsqueeze(0)
            h = stages[0](cur, pos.contiguous(), return_logits=False)
            lg = stages[1](h, pos.contiguous())
            t = int(lg[0, -1].argmax())
            toks.append(t)
            cur = torch.cat([cur, torch.tensor([[t]])], 1)
        assert o == toks, (o, toks)


def _tppp_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.pipeline import SamplingParams
    from tensorlink_amd.parallel.tp import TPPPRunner
    init_distributed(backend="gloo")
    r = TPPPRunner("tiny", rank, world, tp=2, device=torch.device("cpu"),
                   seed=0)
    torch.manual_seed(77)
    ids = torch.randint(0, 1024, (2, 12))
    out = r.generate(ids, SamplingParams(max_new_tokens=5))
    q.put((rank, out.tolist() if out is not None else None))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_tp2_pp2_grid_matches_pp2():
    """2-D TP x PP grid (world=4, tp=2, pp=2): head-sharded stages with
    per-stage TP all-reduces reproduce the pure-PP2 greedy output (same
    per-stage seeded init, sliced)."""
    outs = dict(_run_collect(_tppp_worker, 4, _port(21)))
    # both pipeline replicas' first ranks (0 and 2) return the tokens
    assert outs[0] is not None and outs[2] is not None
    assert outs[0] == outs[2]
    assert outs[1] is None and outs[3] is None

    # pure-PP2 reference (same seeds): single-proc stage composition
    import torch
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 2)
    stages = []
    for rk in range(2):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=rk)
        stages.append(st)
    torch.manual_seed(77)
    ids = torch.randint(0, 1024, (2, 12))
    cur = ids
    for _ in range(5):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).expand(2, -1).contiguous()
        h = stages[0](cur, pos, return_logits=False)
        logits = stages[1](h, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert cur[:, 12:].tolist() == outs[0]


def _dm_tp_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.module import DistributedModel
    m = DistributedModel("tiny", world_size=world, mode="torchrun", tp=2,
                         device=torch.device("cpu"), seed=0)
    torch.manual_seed(88)
    ids = torch.randint(0, 1024, (1, 10))
    if rank == 0:
        out = m.generate(ids, max_new_tokens=4)
        m.shutdown()
        q.put((rank, out.tolist()))
    else:
        m.serve_worker()
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_distributed_model_tp_grid():
    """DistributedModel(tp=2) on a 4-rank torchrun-style world: the user
    API drives the TP x PP grid and returns prompt+tokens on rank 0."""
    outs = dict(_run_collect(_dm_tp_worker, 4, _port(23), n_results=1))
    out = outs[0]
    assert len(out) == 1 and len(out[0]) == 14    # 10 prompt + 4 new


def _cp_train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.cp import CPTrainer
    init_distributed(backend="gloo")
    tr = CPTrainer("tiny", rank, world, device=torch.device("cpu"),
                   seed=13, lr=1e-3)
    torch.manual_seed(91)
    batches = [torch.randint(0, 1024, (2, 24)) for _ in range(3)]
    losses = [tr.train_step(b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_cp2_training_matches_single_rank():
    """CP training: differentiable K/V ring + per-chunk losses + grad
    SUM all-reduce reproduce the single-rank full-sequence loss
    trajectory over 3 optimizer steps."""
    outs = dict(_run_collect(_cp_train_worker, 2, _port(25)))
    assert outs[0] == pytest.approx(outs[1], rel=1e-5)

    import torch
    from tensorlink_amd import ops as tl_ops
    from tensorlink_amd.models.configs import get_config
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.optim import FusedAdamW
    m = build_full_model(get_config("tiny"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=13)
    m.train()
    for p in m.parameters():
        p.requires_grad_(True)
    opt = FusedAdamW(m.parameters(), lr=1e-3, weight_decay=0.01)
    torch.manual_seed(91)
    batches = [torch.randint(0, 1024, (2, 24)) for _ in range(3)]
    ref_losses = []
    for ids in batches:
        B, S = ids.shape
        pos = torch.arange(S, dtype=torch.int32
                           ).unsqueeze(0).expand(B, -1).contiguous()
        opt.zero_grad()
        logits = m.head(m(ids, pos, training=True, return_logits=False))
        loss = tl_ops.causal_lm_loss(logits, ids)
        loss.backward()
        opt.step()
        ref_losses.append(float(loss.detach()))
    assert outs[0] == pytest.approx(ref_losses, rel=2e-3)


def _ep_train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.ep import EPTrainer
    init_distributed(backend="gloo")
    tr = EPTrainer("tiny-moe", rank, world, device=torch.device("cpu"),
                   seed=15, lr=1e-3)
    torch.manual_seed(95)
    batches = [torch.randint(0, 1024, (2, 16)) for _ in range(3)]
    losses = [tr.train_step(b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_ep2_training_matches_single_rank():
    """EP training: differentiable partial-sum all-reduce + router grad
    sum reproduce the single-rank MoE loss trajectory."""
    outs = dict(_run_collect(_ep_train_worker, 2, _port(27)))
    assert outs[0] == pytest.approx(outs[1], rel=1e-5)

    import torch
    from tensorlink_amd import ops as tl_ops
    from tensorlink_amd.models.configs import get_config
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.optim import FusedAdamW
    m = build_full_model(get_config("tiny-moe"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=15)
    m.train()
    for p in m.parameters():
        p.requires_grad_(True)
    opt = FusedAdamW(m.parameters(), lr=1e-3, weight_decay=0.01)
    torch.manual_seed(95)
    batches = [torch.randint(0, 1024, (2, 16)) for _ in range(3)]
    ref_losses = []
    for ids in batches:
        B, S = ids.shape
        pos = torch.arange(S, dtype=torch.int32
                           ).unsqueeze(0).expand(B, -1).contiguous()
        opt.zero_grad()
        logits = m.head(m(ids, pos, training=True, return_logits=False))
        loss = tl_ops.causal_lm_loss(logits, ids)
        loss.backward()
        opt.step()
        ref_losses.append(float(loss.detach()))
    assert outs[0] == pytest.approx(ref_losses, rel=2e-3)


def _tppp_train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.tp import TPPPTrainer
    init_distributed(backend="gloo")
    tr = TPPPTrainer("tiny", rank, world, tp=2,
                     device=torch.device("cpu"), seed=0, lr=1e-3)
    torch.manual_seed(99)
    batches = [torch.randint(0, 1024, (2, 16)) for _ in range(2)]
    losses = [tr.train_step(b, labels=b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


def _pp2_train_ref_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.pipeline import PipelineTrainer
    from tensorlink_amd.parallel.planner import plan_for_world
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", 2, training=True)
    tr = PipelineTrainer(plan, rank, 2, device=torch.device("cpu"),
                         seed=0, lr=1e-3)
    torch.manual_seed(99)
    batches = [torch.randint(0, 1024, (2, 16)) for _ in range(2)]
    losses = [tr.train_step(b, labels=b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_tp2_pp2_training_matches_pp2():
    """TP x PP training: 4-rank tp2 x pp2 grid reproduces the pure-PP2
    loss trajectory (same per-stage seeded init, f/g collectives in the
    sharded projections, 1F1B across stages)."""
    grid = dict(_run_collect(_tppp_train_worker, 4, _port(29)))
    ref = dict(_run_collect(_pp2_train_ref_worker, 2, _port(31)))
    assert grid[0] == pytest.approx(grid[2], rel=1e-5)  # replicas agree
    assert grid[0] == pytest.approx(ref[0], rel=2e-3)


def _h3d_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.tp import Hybrid3DTrainer
    init_distributed(backend="gloo")
    tr = Hybrid3DTrainer("tiny", rank, world, dp=2, tp=2,
                         device=torch.device("cpu"), seed=0, lr=1e-3)
    torch.manual_seed(103)
    full = [torch.randint(0, 1024, (4, 16)) for _ in range(2)]
    shards = [b[tr.dp_rank * 2:(tr.dp_rank + 1) * 2] for b in full]
    losses = [tr.train_step(b, labels=b) for b in shards]
    q.put((rank, (tr.dp_rank, losses)))
    dist.destroy_process_group()


def _pp2_full_ref_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.pipeline import PipelineTrainer
    from tensorlink_amd.parallel.planner import plan_for_world
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", 2, training=True)
    tr = PipelineTrainer(plan, rank, 2, device=torch.device("cpu"),
                         seed=0, lr=1e-3)
    torch.manual_seed(103)
    full = [torch.randint(0, 1024, (4, 16)) for _ in range(2)]
    losses = [tr.train_step(b, labels=b) for b in full]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(600)
def test_dp2_tp2_pp2_matches_pp2_full_batch():
    """3-D grid (8 ranks, dp2 x tp2 x pp2): per-shard losses averaged
    across the DP replicas reproduce the pure-PP2 full-batch loss
    trajectory (grad averaging == mean-reduction on the union batch)."""
    grid = dict(_run_collect(_h3d_worker, 8, _port(33), timeout=400))
    ref = dict(_run_collect(_pp2_full_ref_worker, 2, _port(35)))
    by_dp = {}
    for rank, (dp_rank, losses) in grid.items():
        by_dp.setdefault(dp_rank, losses)
        assert losses == pytest.approx(by_dp[dp_rank], rel=1e-5)
    mean = [(a + b) / 2 for a, b in zip(by_dp[0], by_dp[1])]
    assert mean == pytest.approx(ref[0], rel=2e-3)


def _tp_vp_train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.tp import TPTrainer
    init_distributed(backend="gloo")
    tr = TPTrainer("tiny", rank, world, device=torch.device("cpu"), seed=9,
                   lr=1e-3, vocab_parallel=True)
    assert tr.stage.lm_head.weight.shape[0] == tr.config.vocab_size // world
    torch.manual_seed(41)
    batches = [torch.randint(0, 1024, (2, 24)) for _ in range(3)]
    losses = [tr.train_step(b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_tp2_vocab_parallel_training_matches_single_rank():
    """Vocab-parallel head + Megatron CE (no logits gather): the sharded
    head reproduces the single-rank loss trajectory exactly."""
    outs = dict(_run_collect(_tp_vp_train_worker, 2, _port(37)))
    assert outs[0] == pytest.approx(outs[1], rel=1e-4)

    import torch
    from tensorlink_amd import ops as tl_ops
    from tensorlink_amd.models.configs import get_config
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.optim import FusedAdamW
    m = build_full_model(get_config("tiny"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=9)
    m.train()
    for p in m.parameters():
        p.requires_grad_(True)
    opt = FusedAdamW(m.parameters(), lr=1e-3, weight_decay=0.01)
    torch.manual_seed(41)
    batches = [torch.randint(0, 1024, (2, 24)) for _ in range(3)]
    ref_losses = []
    for ids in batches:
        B, S = ids.shape
        pos = torch.arange(S, dtype=torch.int32
                           ).unsqueeze(0).expand(B, -1).contiguous()
        opt.zero_grad()
        logits = m.head(m(ids, pos, training=True, return_logits=False))
        loss = tl_ops.causal_lm_loss(logits, ids)
        loss.backward()
        opt.step()
        ref_losses.append(float(loss.detach()))
    assert outs[0] == pytest.approx(ref_losses, rel=2e-3)


def _pp_prefix_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.engine.engine import InferenceEngine
    from tensorlink_amd.parallel.comm import init_distributed
    init_distributed(backend="gloo")
    eng = InferenceEngine(rank=rank, world=world, device=torch.device("cpu"))
    if rank != 0:
        eng.worker_loop()
        return
    eng.load_model("tiny", continuous=True, max_slots=4, max_ctx=512,
                   prefill_chunk=64, prefix_caching=True)
    b = eng.jobs["tiny"].batcher
    torch.manual_seed(47)
    prompt = torch.randint(0, 1024, (300,))
    out1 = b.submit(prompt.clone(), max_new_tokens=6).result(timeout=120)
    out2 = b.submit(prompt.clone(), max_new_tokens=6).result(timeout=120)
    hits = b.cache.hits
    import time
    for _ in range(200):
        if (b.cache.allocator.n_free + len(b.cache.lru)
                == b.cache.allocator.n_pages):
            break
        time.sleep(0.02)
    drained = (b.cache.allocator.n_free + len(b.cache.lru)
               == b.cache.allocator.n_pages)
    eng.unload_model("tiny")
    eng.shutdown()
    q.put((rank, (out1, out2, hits, drained)))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_pp2_prefix_caching():
    """Prefix caching across a 2-stage pipeline: admissions ride the
    command stream, so follower allocators adopt/register the same pages
    in lockstep; the repeat request reuses 2 pages and outputs match."""
    outs = dict(_run_collect(_pp_prefix_worker, 2, _port(39), n_results=1))
    out1, out2, hits, drained = outs[0]
    assert out1 == out2
    assert hits == 256
    assert drained


def _tppp_vp_train_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.tp import TPPPTrainer
    init_distributed(backend="gloo")
    tr = TPPPTrainer("tiny", rank, world, tp=2, device=torch.device("cpu"),
                     seed=0, lr=1e-3, vocab_parallel=True)
    if tr.trainer.stage.has_head:
        assert tr.trainer.stage.lm_head.weight.shape[0] == \
            tr.config.vocab_size // 2
    torch.manual_seed(99)
    batches = [torch.randint(0, 1024, (2, 16)) for _ in range(2)]
    losses = [tr.train_step(b, labels=b) for b in batches]
    q.put((rank, losses))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_tp2_pp2_vocab_parallel_training():
    """TP x PP with a vocab-sharded head on the last stage: the Megatron
    gather-free CE reproduces the pure-PP2 loss trajectory."""
    grid = dict(_run_collect(_tppp_vp_train_worker, 4, _port(41)))
    ref = dict(_run_collect(_pp2_train_ref_worker, 2, _port(43)))
    assert grid[0] == pytest.approx(grid[2], rel=1e-5)
    assert grid[0] == pytest.approx(ref[0], rel=2e-3)


def _cp_qk_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.cp import CPRunner
    init_distributed(backend="gloo")
    r = CPRunner("tiny-qwen3", rank, world, device=torch.device("cpu"),
                 seed=19)
    torch.manual_seed(57)
    ids = torch.randint(0, 1024, (1, 24))
    out = r.generate(ids, max_new_tokens=4)
    q.put((rank, out.tolist()))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_cp2_qwen3_qk_norm():
    """CP honors Qwen3's per-head qk-norm (prefill + decode) — matches
    the single-rank model."""
    outs = dict(_run_collect(_cp_qk_worker, 2, _port(45)))
    assert outs[0] == outs[1]

    import torch
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.models.configs import get_config
    m = build_full_model(get_config("tiny-qwen3"))
    init_random_stage(m, device="cpu", dtype=torch.float32, seed=19)
    torch.manual_seed(57)
    ids = torch.randint(0, 1024, (1, 24))
    cur = ids
    for _ in range(4):
        pos = torch.arange(cur.shape[1]).unsqueeze(0).contiguous()
        logits = m(cur, pos)
        cur = torch.cat([cur, logits[:, -1].argmax(-1, keepdim=True)], 1)
    assert cur[:, 24:].tolist() == outs[0]


def _pp4_batch_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.engine.engine import InferenceEngine
    from tensorlink_amd.parallel.comm import init_distributed
    init_distributed(backend="gloo")
    eng = InferenceEngine(rank=rank, world=world, device=torch.device("cpu"))
    if rank != 0:
        eng.worker_loop()
        return
    eng.load_model("tiny", continuous=True, max_slots=3, max_ctx=256,
                   prefill_chunk=32, prefix_caching=True)
    b = eng.jobs["tiny"].batcher
    torch.manual_seed(61)
    prompts = [torch.randint(0, 1024, (n,)) for n in (40, 150, 150)]
    prompts[2] = prompts[1].clone()
    reqs = [b.submit(p.clone(), max_new_tokens=6) for p in prompts[:2]]
    outs = [rq.result(timeout=180) for rq in reqs]
    # duplicate prompt AFTER the original registered its pages
    r3 = b.submit(prompts[2].clone(), max_new_tokens=6)
    outs.append(r3.result(timeout=180))
    hits = b.cache.hits
    eng.unload_model("tiny")
    eng.shutdown()
    q.put((rank, ([p.tolist() for p in prompts], outs, hits)))
    dist.destroy_process_group()


@pytest.mark.timeout(600)
def test_pp4_continuous_batching():
    """4-stage pipeline batcher (deep pipeline + chunked prefill +
    prefix reuse) reproduces serial greedy outputs."""
    outs = dict(_run_collect(_pp4_batch_worker, 4, _port(47),
                             n_results=1, timeout=400))
    prompts, results, hits = outs[0]
    assert hits >= 128          # repeated 150-token prompt reused a page

    import torch
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 4)
    stages = []
    for rk in range(4):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=rk)
        stages.append(st)
    for p, o in zip(prompts, results):
        cur = torch.tensor(p, dtype=torch.int64).unsqueeze(0)
        toks = []
        for _ in range(6):
            pos = torch.arange(cur.shape[1]).unsqueeze(0).contiguous()
            h = cur
            for st in stages[:-1]:
                h = st(h, pos, return_logits=False)
            lg = stages[-1](h, pos)
            t = int(lg[0, -1].argmax())
            toks.append(t)
            cur = torch.cat([cur, torch.tensor([[t]])], 1)
        assert o == toks, (o, toks)


def _lora_pp_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.pipeline import PipelineTrainer
    from tensorlink_amd.parallel.planner import plan_for_world
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", 2, training=True)
    t = PipelineTrainer(plan, rank, 2, device=torch.device("cpu"),
                        seed=0, lr=5e-3, lora_r=4)
    base = {k: v.clone() for k, v in t.stage.state_dict().items()
            if ".base.weight" in k}
    torch.manual_seed(31)
    losses = []
    for _ in range(6):
        b = torch.randint(0, 1024, (2, 16))
        losses.append(t.train_step(b, labels=b))
    frozen = all(torch.equal(v, t.stage.state_dict()[k])
                 for k, v in base.items())
    q.put((rank, (losses, frozen,
                  t.optimizer.flat_param.numel())))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_lora_across_pipeline():
    """LoRA over a 2-stage pipeline: adapters train (loss falls), base
    weights stay frozen, optimizer state is tiny."""
    outs = dict(_run_collect(_lora_pp_worker, 2, _port(49)))
    for rank, (losses, frozen, n_opt) in outs.items():
        assert losses[-1] < losses[0]
        assert frozen
        assert n_opt < 100_000          # adapters only (full stage ~1.5M)


def _family_par_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.ep import EPRunner
    from tensorlink_amd.parallel.pipeline import SamplingParams
    from tensorlink_amd.parallel.tp import TPRunner
    init_distributed(backend="gloo")
    r = EPRunner("tiny-qwen3-moe", rank, world,
                 device=torch.device("cpu"), seed=4)
    torch.manual_seed(6)
    ids = torch.randint(0, 1024, (1, 10))
    out = r.generate(ids, SamplingParams(max_new_tokens=4))
    r2 = TPRunner("tiny-qwen3", rank, world, device=torch.device("cpu"),
                  seed=4)
    out2 = r2.generate(ids, SamplingParams(max_new_tokens=4))
    q.put((rank, (out.tolist(), out2.tolist())))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_ep_tp_on_new_families():
    """EP handles Qwen3-MoE's per-expert width; TP shards qk-norm heads
    (Qwen3) — both reproduce single-rank outputs."""
    outs = dict(_run_collect(_family_par_worker, 2, _port(51)))
    assert outs[0] == outs[1]

    import torch
    from tensorlink_amd.models.configs import get_config
    from tensorlink_amd.models.dense import build_full_model
    from tensorlink_amd.models.loader import init_random_stage
    for preset, got in (("tiny-qwen3-moe", outs[0][0]),
                        ("tiny-qwen3", outs[0][1])):
        m = build_full_model(get_config(preset))
        init_random_stage(m, device="cpu", dtype=torch.float32, seed=4)
        torch.manual_seed(6)
        cur = torch.randint(0, 1024, (1, 10))
        for _ in range(4):
            pos = torch.arange(cur.shape[1]).unsqueeze(0).contiguous()
            lg = m(cur, pos)
            cur = torch.cat([cur, lg[:, -1].argmax(-1, keepdim=True)], 1)
        assert cur[:, 10:].tolist() == got


def _pp_spec_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.engine.batcher import PPContinuousBatcher
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.planner import plan_for_world
    from tensorlink_amd.parallel.pipeline import PipelineRunner
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", world)
    r = PipelineRunner(plan, rank, world, device=torch.device("cpu"),
                       seed=10)
    b = PPContinuousBatcher(r, max_slots=3, max_ctx=256, prefill_chunk=16,
                            speculative=True)
    if rank != 0:
        b.serve_follower()
        dist.destroy_process_group()
        return
    b.start()
    torch.manual_seed(19)
    # seed 10's tiny decode loops => proposals get accepted
    prompts = [torch.randint(0, 1024, (16,)) for _ in range(2)]
    reqs = [b.submit(p.clone(), max_new_tokens=24) for p in prompts]
    outs = [rq.result(timeout=120) for rq in reqs]
    steps, acc = b.steps, b.spec_accepted
    b.stop()
    q.put((rank, ([p.tolist() for p in prompts], outs, steps, acc)))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_pp2_speculative_batching_matches_serial():
    """Speculation through the PP batcher: rank 0 proposes via prompt
    lookup, every rank executes the ragged verify rows in lockstep, and
    the output equals non-speculative serial greedy with fewer
    scheduler steps and accepted proposals."""
    outs = dict(_run_collect(_pp_spec_worker, 2, _port(23), n_results=1))
    prompts, results, steps, acc = outs[0]
    assert acc > 0, "no proposals accepted"
    assert steps < 2 * 24         # multi-token emission happened

    import torch
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 2)
    stages = []
    for rk in range(2):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=10 + rk)
        stages.append(st)
    for p, o in zip(prompts, results):
        cur = torch.tensor(p, dtype=torch.int64).unsqueeze(0)
        toks = []
        for _ in range(24):
            pos = torch.arange(cur.shape[1]).unsqueeze(0)
            h = stages[0](cur, pos.contiguous(), return_logits=False)
            lg = stages[1](h, pos.contiguous())
            t = int(lg[0, -1].argmax())
            toks.append(t)
            cur = torch.cat([cur, torch.tensor([[t]])], 1)
        assert o == toks, (o, toks)


def _pp_compose_worker(rank, world, port, q):
    sys.path.insert(0, REPO)
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port))
    import torch
    import torch.distributed as dist
    from tensorlink_amd.engine.batcher import PPContinuousBatcher
    from tensorlink_amd.parallel.comm import init_distributed
    from tensorlink_amd.parallel.planner import plan_for_world
    from tensorlink_amd.parallel.pipeline import PipelineRunner
    init_distributed(backend="gloo")
    plan = plan_for_world("tiny", world)
    r = PipelineRunner(plan, rank, world, device=torch.device("cpu"),
                       seed=10)
    b = PPContinuousBatcher(r, max_slots=2, max_ctx=512, prefill_chunk=64,
                            prefix_caching=True, speculative=True)
    if rank != 0:
        b.serve_follower()
        dist.destroy_process_group()
        return
    b.start()
    torch.manual_seed(19)
    p = torch.randint(0, 1024, (150,))
    o1 = b.submit(p.clone(), max_new_tokens=30).result(timeout=120)
    o2 = b.submit(p.clone(), max_new_tokens=30).result(timeout=120)
    hits, acc = b.cache.hits, b.spec_accepted
    b.stop()
    q.put((rank, (p.tolist(), o1, o2, hits, acc)))
    dist.destroy_process_group()


@pytest.mark.timeout(300)
def test_pp2_spec_prefix_chunked_composition():
    """The earlier failing composition (chunked prefill + prefix caching
    + speculation) on the PP batcher: repeat prompt reuses pages, the
    lockstep ragged verify accepts proposals, and output equals serial
    greedy."""
    outs = dict(_run_collect(_pp_compose_worker, 2, _port(27), n_results=1))
    prompt, o1, o2, hits, acc = outs[0]
    # (acceptance count is sequence-dependent — this prompt's output has
    # no 3-gram repeats; acc > 0 is pinned by the dedicated spec test)
    assert o1 == o2 and hits == 128

    import torch
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 2)
    stages = []
    for rk in range(2):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=10 + rk)
        stages.append(st)
    cur = torch.tensor(prompt, dtype=torch.int64).unsqueeze(0)
    toks = []
    for _ in range(30):
        pos = torch.arange(cur.shape[1]).unsqueeze(0)
        h = stages[0](cur, pos.contiguous(), return_logits=False)
        lg = stages[1](h, pos.contiguous())
        t = int(lg[0, -1].argmax())
        toks.append(t)
        cur = torch.cat([cur, torch.tensor([[t]])], 1)
    assert o1 == toks, (o1, toks)


@pytest.mark.timeout(300)
def test_pp4_speculative_batching():
    """The lockstep ragged-verify protocol generalizes past 2 stages:
    pp4 speculative batching equals the 4-stage chained reference."""
    outs = dict(_run_collect(_pp_spec_worker, 4, _port(29), n_results=1))
    prompts, results, steps, acc = outs[0]
    # acceptance depends on the sequence having n-gram repeats (pinned
    # by the pp2 test); here the 4-stage lockstep protocol + equality
    # are the subject

    import torch
    from tensorlink_amd.models.dense import build_stage
    from tensorlink_amd.models.loader import init_random_stage
    from tensorlink_amd.parallel.planner import plan_for_world
    plan = plan_for_world("tiny", 4)
    stages = []
    for rk in range(4):
        st = build_stage(plan.config, plan.stage_for_rank(rk))
        init_random_stage(st, dtype=torch.float32, seed=10 + rk)
        stages.append(st)
    for p, o in zip(prompts, results):
        cur = torch.tensor(p, dtype=torch.int64).unsqueeze(0)
        toks = []
        for _ in range(24):
            pos = torch.arange(cur.shape[1]).unsqueeze(0).contiguous()
            h = cur
            for st in stages[:-1]:
                h = st(h, pos, return_logits=False)
            lg = stages[-1](h, pos)
            t = int(lg[0, -1].argmax())
            toks.append(t)
            cur = torch.cat([cur, torch.tensor([[t]])], 1)
        assert o == toks, (o, toks)
