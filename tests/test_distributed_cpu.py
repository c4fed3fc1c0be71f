"""Multi-process (gloo, CPU) model-parallel pipeline and data-parallel runs
must reproduce the single-process scores exactly."""
import os
import pickle
import socket

import numpy as np
import pytest
import torch
import torch.multiprocessing as mp


def _close(a, b):
    # fp32 CPU GEMM reductions depend on the thread count: allow 1-ulp fp16 differences
    return a.shape == b.shape and np.abs(a.astype(np.float32) - b.astype(np.float32)).max() < 1e-5


def _port():
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    p = s.getsockname()[1]
    s.close()
    return p


def _worker(rank, world, port, path, prompts, lnps, dp, storage, out_dir, budget, pkv=False,
            stages="round_robin"):
    os.environ.update({"RANK": str(rank), "WORLD_SIZE": str(world), "LOCAL_RANK": str(rank),
                       "MASTER_ADDR": "127.0.0.1", "MASTER_PORT": str(port)})
    torch.set_num_threads(1)
    from flexible_llm_sharding_amd.config import ModelConfig
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.parallel.comm import Comm
    from flexible_llm_sharding_amd.runtime.stream import FileLayerSource
    from flexible_llm_sharding_amd.utils.tokenizer import load_tokenizer
    comm = Comm.from_env("cpu", timeout_s=120)
    cfg = ModelConfig.from_pretrained(path)
    tok = load_tokenizer(path)
    r = ShardedRunner(cfg, FileLayerSource(cfg, path), "cpu", tok, layer_num_per_shard=lnps,
                      storage_location=storage, disk_folder=os.path.join(out_dir, f"spill{rank}"),
                      comm=comm, data_parallel=dp, token_budget=budget, prefix_kv_cache=pkv,
                      pipeline_stages=stages)
    if stages == "contiguous" and not dp:
        flat = [i for sh in r.my_shards for i in sh]
        assert flat == list(range(flat[0], flat[0] + len(flat)))          # one contiguous stage
    if dp:
        idx = np.array_split(np.arange(len(prompts)), world)[rank]
        mine = [prompts[i] for i in idx]
    else:
        mine = prompts
    outs = r(mine)
    # run twice: state must be clean between calls (reference races here)
    outs2 = r(mine)
    for a, b in zip(outs, outs2):
        assert (a is None and b is None) or (_close(a, b) if pkv else np.array_equal(a, b))
    if pkv:
        assert r.stats["prefix_cached"] == 1.0 and r.prefix_cache.hits == 1
    allv = comm.gather_scores(outs, dst=0)
    resumed = comm.gather_object(r.stats["resumed_from_shard"], dst=0)
    if rank == 0:
        with open(os.path.join(out_dir, "out.pkl"), "wb") as f:
            pickle.dump(allv, f)
        with open(os.path.join(out_dir, "resumed.pkl"), "wb") as f:
            pickle.dump(resumed, f)
    comm.destroy()


@pytest.fixture(scope="module")
def single(tiny_model):
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.runtime.stream import FileLayerSource
    from flexible_llm_sharding_amd.utils.synthetic import synthetic_prompts
    from flexible_llm_sharding_amd.utils.tokenizer import load_tokenizer
    path, cfg = tiny_model
    prompts = synthetic_prompts(7, 25, 3, 6, cfg.vocab_size, seed=21, vary=True)
    out = ShardedRunner(cfg, FileLayerSource(cfg, path), "cpu", load_tokenizer(path))(prompts)
    return path, prompts, out


@pytest.mark.parametrize("world,lnps,storage,budget,stages", [
    (2, 1, "cpu", 40, "round_robin"), (3, 1, "gpu", 30, "round_robin"), (2, 2, "disk", 1000, "round_robin"),
    (4, 1, "cpu", 60, "round_robin"), (2, 1, "cpu", 40, "contiguous"), (3, 2, "gpu", 30, "contiguous")])
def test_model_parallel_pipeline(single, tmp_path, world, lnps, storage, budget, stages):
    path, prompts, ref = single
    mp.start_processes(_worker, args=(world, _port(), path, prompts, lnps, False, storage, str(tmp_path), budget,
                                      False, stages),
                       nprocs=world, start_method="spawn", join=True)
    allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
    owner = [v for v in allv if v and v[0] is not None]
    assert len(owner) == 1
    for a, b in zip(owner[0], ref):
        assert _close(a, b)


@pytest.mark.parametrize("world", [2, 3])
def test_data_parallel(single, tmp_path, world):
    path, prompts, ref = single
    mp.start_processes(_worker, args=(world, _port(), path, prompts, 1, True, "cpu", str(tmp_path), 50),
                       nprocs=world, start_method="spawn", join=True)
    allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
    got = sum(allv, [])
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        assert _close(a, b)


def _dp_shard_worker(rank, world, port, path, prompts, lnps, out_dir, resume_dir=None, fault="", weights="host"):
    if fault:
        os.environ["FLS_FAULT"] = fault
    os.environ.update({"RANK": str(rank), "WORLD_SIZE": str(world), "LOCAL_RANK": str(rank),
                       "MASTER_ADDR": "127.0.0.1", "MASTER_PORT": str(port)})
    torch.set_num_threads(1)
    from types import SimpleNamespace
    from flexible_llm_sharding_amd.config import ModelConfig
    from flexible_llm_sharding_amd.parallel.comm import Comm
    from flexible_llm_sharding_amd.parallel.data_parallel import build_dp_sharded_runner
    from flexible_llm_sharding_amd.utils.tokenizer import load_tokenizer
    comm = Comm.from_env("cpu", timeout_s=120)
    cfg = ModelConfig.from_pretrained(path)
    args = SimpleNamespace(model_path=path, layer_num_per_shard=lnps, storage_location="cpu",
                           disk_folder=out_dir, max_activation_in_cpu=100, prefix_attention="bidirectional",
                           token_budget=50, resident=False, dtype=None, verbose=False,
                           resume_dir=resume_dir, checkpoint_every=2)
    r = build_dp_sharded_runner(args, cfg, "cpu", comm, load_tokenizer(path), weight_cache=weights)
    assert r.prefetcher.__class__.__name__ == "AllGatherPrefetcher"
    assert r.prefetcher.streaming == (weights == "stream")
    idx = np.array_split(np.arange(len(prompts)), world)[rank]
    outs = r([prompts[i] for i in idx])
    allv = comm.gather_scores(outs, dst=0)
    resumed = comm.gather_object(r.stats["resumed_from_shard"], dst=0)
    if rank == 0:
        with open(os.path.join(out_dir, "out.pkl"), "wb") as f:
            pickle.dump(allv, f)
        with open(os.path.join(out_dir, "resumed.pkl"), "wb") as f:
            pickle.dump(resumed, f)
    comm.destroy()


@pytest.mark.parametrize("world,lnps", [(2, 1), (3, 2)])
def test_data_parallel_sharded_weights(single, tmp_path, world, lnps):
    path, prompts, ref = single
    mp.start_processes(_dp_shard_worker, args=(world, _port(), path, prompts, lnps, str(tmp_path)),
                       nprocs=world, start_method="spawn", join=True)
    got = sum(pickle.load(open(tmp_path / "out.pkl", "rb")), [])
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        assert _close(a, b)


def _fault_worker(rank, world, port, path, prompts, out_dir):
    os.environ["FLS_FAULT"] = "1:1"
    _worker(rank, world, port, path, prompts, 1, False, "gpu", out_dir, 40)


def test_rank_failure_terminates_job(single, tmp_path):
    """A rank dying mid-pipeline must end the whole job (no peer left blocked in recv)."""
    import time
    path, prompts, ref = single
    t0 = time.time()
    with pytest.raises(Exception) as ei:
        mp.start_processes(_fault_worker, args=(2, _port(), path, prompts, str(tmp_path)), nprocs=2,
                           start_method="spawn", join=True)
    assert "FLS_FAULT" in str(ei.value) or "exited" in str(ei.value) or "ProcessRaised" in type(ei.value).__name__
    assert time.time() - t0 < 120


def test_data_parallel_resume_after_rank_fault(single, tmp_path):
    """DP + --resume_dir: rank 1 dies at shard 3; the relaunch resumes every rank at shard 2."""
    path, prompts, ref = single
    ck = str(tmp_path / "ck")
    with pytest.raises(Exception):
        mp.start_processes(_dp_shard_worker, args=(2, _port(), path, prompts, 1, str(tmp_path), ck, "1:3"),
                           nprocs=2, start_method="spawn", join=True)
    mp.start_processes(_dp_shard_worker, args=(2, _port(), path, prompts, 1, str(tmp_path), ck, ""),
                       nprocs=2, start_method="spawn", join=True)
    assert pickle.load(open(tmp_path / "resumed.pkl", "rb")) == [2.0, 2.0]
    got = sum(pickle.load(open(tmp_path / "out.pkl", "rb")), [])
    for a, b in zip(got, ref):
        assert _close(a, b)


@pytest.mark.parametrize("world,dp", [(3, False), (2, True)])
def test_prefix_kv_cache_distributed(single, tmp_path, world, dp):
    """Second call reuses every rank's prefix K/V (MP ranks agree on the cached packing)."""
    path, prompts, ref = single
    mp.start_processes(_worker, args=(world, _port(), path, prompts, 1, dp, "cpu", str(tmp_path), 40, True),
                       nprocs=world, start_method="spawn", join=True)
    allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
    got = sum(allv, []) if dp else [v for v in allv if v and v[0] is not None][0]
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        assert _close(a, b)


def _mp_resume_worker(rank, world, port, path, prompts, out_dir, resume_dir, fault, storage):
    if fault:
        os.environ["FLS_FAULT"] = fault
    os.environ.update({"RANK": str(rank), "WORLD_SIZE": str(world), "LOCAL_RANK": str(rank),
                       "MASTER_ADDR": "127.0.0.1", "MASTER_PORT": str(port)})
    torch.set_num_threads(1)
    from flexible_llm_sharding_amd.config import ModelConfig
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.parallel.comm import Comm
    from flexible_llm_sharding_amd.runtime.stream import FileLayerSource
    from flexible_llm_sharding_amd.utils.tokenizer import load_tokenizer
    comm = Comm.from_env("cpu", timeout_s=60)
    cfg = ModelConfig.from_pretrained(path)
    r = ShardedRunner(cfg, FileLayerSource(cfg, path), "cpu", load_tokenizer(path), layer_num_per_shard=1,
                      storage_location=storage, disk_folder=os.path.join(out_dir, f"spill{rank}"), comm=comm,
                      token_budget=40, resume_dir=resume_dir, checkpoint_every=2)
    outs = r(prompts)
    allv = comm.gather_scores(outs, dst=0)
    resumed = comm.gather_object(r.stats["resumed_from_shard"], dst=0)
    if rank == 0:
        with open(os.path.join(out_dir, "out.pkl"), "wb") as f:
            pickle.dump(allv, f)
        with open(os.path.join(out_dir, "resumed.pkl"), "wb") as f:
            pickle.dump(resumed, f)
    comm.destroy()


@pytest.fixture(scope="module")
def deeper(tmp_path_factory):
    """6 decoder layers: a 2-rank round-robin pipeline has 5 shards per rank."""
    from flexible_llm_sharding_amd.config import preset
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.runtime.stream import FileLayerSource
    from flexible_llm_sharding_amd.utils.synthetic import synthetic_prompts, write_synthetic_checkpoint
    from flexible_llm_sharding_amd.utils.tokenizer import load_tokenizer
    cfg = preset("tiny", num_hidden_layers=6)
    path = str(tmp_path_factory.mktemp("deep"))
    write_synthetic_checkpoint(cfg, path, seed=2, std=0.05)
    prompts = synthetic_prompts(7, 25, 3, 6, cfg.vocab_size, seed=22, vary=True)
    out = ShardedRunner(cfg, FileLayerSource(cfg, path), "cpu", load_tokenizer(path))(prompts)
    return path, prompts, out


@pytest.mark.parametrize("storage", ["cpu", "disk"])
def test_model_parallel_resume_after_rank_fault(deeper, tmp_path, storage):
    """MP + --resume_dir: each stage checkpoints its inputs every 2 global shards; rank 1 dies
    entering its 4th shard; the relaunch restarts every rank at the latest stage boundary whose
    consumer holds its inputs (rank 0 resumes mid-pipeline, rank 1 after it) and matches a clean run.
    Received activations drain through the receiver thread into the chosen storage."""
    path, prompts, ref = deeper
    ck = str(tmp_path / "ck")
    with pytest.raises(Exception):
        mp.start_processes(_mp_resume_worker, args=(2, _port(), path, prompts, str(tmp_path), ck, "1:3", storage),
                           nprocs=2, start_method="spawn", join=True)
    assert any(n.startswith("step") for n in os.listdir(os.path.join(ck, "rank0")))
    mp.start_processes(_mp_resume_worker, args=(2, _port(), path, prompts, str(tmp_path), ck, "", storage),
                       nprocs=2, start_method="spawn", join=True)
    resumed = pickle.load(open(tmp_path / "resumed.pkl", "rb"))
    assert resumed[0] >= 2 and resumed[1] >= 2          # layer 4 or 6 boundary: both ranks skip shards
    allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
    owner = [v for v in allv if v and v[0] is not None]
    assert len(owner) == 1
    for a, b in zip(owner[0], ref):
        assert _close(a, b)
    assert not os.path.exists(ck) or not os.listdir(ck)   # cleared once the run completes


@pytest.fixture(scope="module")
def moe_single(tmp_path_factory):
    from flexible_llm_sharding_amd.config import preset
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.runtime.stream import FileLayerSource
    from flexible_llm_sharding_amd.utils.synthetic import synthetic_prompts, write_synthetic_checkpoint
    from flexible_llm_sharding_amd.utils.tokenizer import load_tokenizer
    cfg = preset("tiny-mixtral", num_hidden_layers=3)
    path = str(tmp_path_factory.mktemp("moe") / "m")
    write_synthetic_checkpoint(cfg, path, seed=31, std=0.05)
    prompts = synthetic_prompts(5, 25, 3, 6, cfg.vocab_size, seed=32, vary=True)
    out = ShardedRunner(cfg, FileLayerSource(cfg, path), "cpu", load_tokenizer(path))(prompts)
    return path, prompts, out


@pytest.mark.parametrize("mode", ["mp", "dp_sharded"])
def test_moe_model_parallel_and_data_parallel(moe_single, tmp_path, mode):
    """A Mixtral-structured model (router + experts in the layer image) through the pipeline and
    the data-parallel all-gather of 1/G byte ranges: same scores as one process."""
    path, prompts, ref = moe_single
    if mode == "mp":
        mp.start_processes(_worker, args=(2, _port(), path, prompts, 1, False, "cpu", str(tmp_path), 40),
                           nprocs=2, start_method="spawn", join=True)
        allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
        got = [v for v in allv if v and v[0] is not None][0]
    else:
        mp.start_processes(_dp_shard_worker, args=(2, _port(), path, prompts, 1, str(tmp_path)),
                           nprocs=2, start_method="spawn", join=True)
        got = sum(pickle.load(open(tmp_path / "out.pkl", "rb")), [])
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        assert _close(a, b)


def _p2p_warmup_worker(rank, world, port, edges, out_dir):
    os.environ.update({"RANK": str(rank), "WORLD_SIZE": str(world), "LOCAL_RANK": str(rank),
                       "MASTER_ADDR": "127.0.0.1", "MASTER_PORT": str(port)})
    from flexible_llm_sharding_amd.parallel.comm import Comm
    comm = Comm.from_env("cpu", timeout_s=60)
    comm.setup_p2p_edges(edges)
    comm.warmup_p2p()
    comm.warmup_p2p()                      # idempotent: a second chain matches up the same way
    comm.barrier()
    with open(os.path.join(out_dir, f"ok{rank}"), "w") as f:
        f.write("ok")
    comm.destroy()


@pytest.mark.parametrize("world,edges", [(2, [(0, 1), (1, 0)]), (3, [(0, 1), (1, 2), (2, 0), (2, 1)])])
def test_p2p_warmup_chain_completes(tmp_path, world, edges):
    """Comm.warmup_p2p (run before a VRAM cap measures device memory in model parallel): every
    rank walks the directed hand-off edges in one order and finishes each before the next, so the
    chain completes for edges in both directions and across more than two ranks."""
    mp.spawn(_p2p_warmup_worker, args=(world, _port(), edges, str(tmp_path)), nprocs=world, join=True)
    assert sorted(os.listdir(tmp_path)) == [f"ok{r}" for r in range(world)]


def _gather_worker(rank, world, port, out_dir):
    os.environ.update({"RANK": str(rank), "WORLD_SIZE": str(world), "LOCAL_RANK": str(rank),
                       "MASTER_ADDR": "127.0.0.1", "MASTER_PORT": str(port)})
    import json
    from flexible_llm_sharding_amd.parallel.comm import Comm
    comm = Comm.from_env("cpu", timeout_s=60)

    def scores(r):
        g = np.random.default_rng(r)
        outs = [g.random((3 + i, 1, 1000)).astype(np.float16) for i in range(3)]
        if r % 2 == 1:
            outs.insert(1, None)                 # a prompt this rank does not own (model parallel)
        return outs
    got = comm.gather_scores(scores(rank), dst=0)
    if rank == 0:
        assert len(got) == world
        for r in range(world):
            want = scores(r)
            assert len(got[r]) == len(want)
            for a, b in zip(got[r], want):
                assert (a is None and b is None) or np.array_equal(a, b)
    else:
        assert got is None
    with open(os.path.join(out_dir, f"stats{rank}.json"), "w") as f:
        json.dump(comm.gather_stats, f)
    comm.destroy()


def test_gather_scores_memory_does_not_grow_with_world(tmp_path):
    """Rank-0 score return (Comm.gather_scores: one packed fp16 tensor + shapes per rank, after a
    fixed-size header): the bytes a rank other than 0 stages and sends are its own scores, the
    same at world 2 and 4 (all_gather_object sent every rank's scores to every rank)."""
    import json
    staged = {}
    for world in (2, 4):
        d = tmp_path / f"w{world}"
        d.mkdir()
        mp.spawn(_gather_worker, args=(world, _port(), str(d)), nprocs=world, join=True)
        st = {r: json.load(open(d / f"stats{r}.json")) for r in range(world)}
        own = (3 + 4 + 5) * 1000 * 2
        for r in range(1, world):
            assert st[r]["staged_bytes"] == st[r]["sent_bytes"] == own
            assert st[r]["received_bytes"] == 0
        assert st[0]["received_bytes"] == (world - 1) * own
        staged[world] = st[1]["staged_bytes"]
    assert staged[2] == staged[4]


# ------------------------------------------------------------------ world 8 (the driver's node)
@pytest.mark.parametrize("stages", ["round_robin", "contiguous"])
def test_model_parallel_world8(deeper, tmp_path, stages):
    """Eight pipeline ranks, the size of the node the driver's scaling run uses.  Round robin: 6
    decoder layers + embed / norm / head = 9 layers -> ceil(9 / 8) * 8 = 16 shards, 7 of them
    padded EMPTY (utils.py:150-153), so some ranks own only empty shards in the second round and
    the wrap-around edge 7 -> 0 carries a layer; contiguous: one block per rank, several ranks of
    a single layer.  Scores equal the one-process run."""
    from flexible_llm_sharding_amd.parallel.planner import make_plan
    path, prompts, ref = deeper
    plans = [make_plan(9, 1, 8, r, False, stages) for r in range(8)]
    if stages == "round_robin":
        assert sum(1 for p in plans for sh in p.my_shards if not len(sh)) == 7
    assert sorted(i for p in plans for sh in p.my_shards for i in sh) == list(range(9))
    mp.start_processes(_worker, args=(8, _port(), path, prompts, 1, False, "cpu", str(tmp_path), 40, False, stages),
                       nprocs=8, start_method="spawn", join=True)
    allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
    owner = [v for v in allv if v and v[0] is not None]
    assert len(owner) == 1
    for a, b in zip(owner[0], ref):
        assert _close(a, b)


@pytest.mark.parametrize("weights", ["host", "stream"])
def test_data_parallel_sharded_world8(single, tmp_path, weights):
    """Eight data-parallel ranks with 1/8-sliced weights all-gathered per layer (pinned slices, or
    streamed from the layer files by each rank's loader thread with the gathers issued from the
    main thread in program order); 7 prompts, so rank 7 has none and still joins every gather."""
    path, prompts, ref = single
    assert len(prompts) < 8
    mp.start_processes(_dp_shard_worker, args=(8, _port(), path, prompts, 1, str(tmp_path), None, "", weights),
                       nprocs=8, start_method="spawn", join=True)
    allv = pickle.load(open(tmp_path / "out.pkl", "rb"))
    assert allv[7] == []
    got = sum(allv, [])
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        assert _close(a, b)


def test_data_parallel_resume_world8(single, tmp_path):
    """DP over 8 ranks + --resume_dir: rank 5 dies entering shard 3; the relaunch resumes every rank
    at shard 2 (the latest checkpoint all 8 hold) and matches the one-process run."""
    path, prompts, ref = single
    ck = str(tmp_path / "ck")
    with pytest.raises(Exception):
        mp.start_processes(_dp_shard_worker, args=(8, _port(), path, prompts, 1, str(tmp_path), ck, "5:3"),
                           nprocs=8, start_method="spawn", join=True)
    mp.start_processes(_dp_shard_worker, args=(8, _port(), path, prompts, 1, str(tmp_path), ck, ""),
                       nprocs=8, start_method="spawn", join=True)
    assert pickle.load(open(tmp_path / "resumed.pkl", "rb")) == [2.0] * 8
    got = sum(pickle.load(open(tmp_path / "out.pkl", "rb")), [])
    for a, b in zip(got, ref):
        assert _close(a, b)
