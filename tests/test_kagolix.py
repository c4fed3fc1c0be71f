"""Kagolix through the framework (config registry, weight images, sequence state cache, step
scheduler, kernels) against the plain float64 oracle in ``kagolix_oracle.py``.

Every test runs on the CPU backend (plain PyTorch ops) and, marked ``gpu``, on the HIP kernels.  The
models are tiny and random; fp32 matrix products make the comparison sharp (a window one token off,
a lost state or a wrong page shows as an error thousands of times the tolerance), and one test runs
the bf16 mode.  Attention layers use a large score scale so that the softmax is peaked: a key that
is wrongly seen or missed then moves the output by much more than rounding."""
import json
import pickle

import numpy as np
import pytest
import torch

import kagolix_util as ku
from conftest import gpu_available
from flexible_llm_sharding_amd.runtime.batch import StepEntry
from flexible_llm_sharding_amd.serve import generate, load_runner

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
TOL = 2e-4          # fp32 products against float64, relative to a logit row's spread


@pytest.fixture(autouse=True)
def _need_gpu(request):
    params = getattr(getattr(request.node, "callspec", None), "params", {})
    if "cuda" in str(params.get("device", "")) and not gpu_available():
        pytest.skip("no GPU")


def build(tmp_path, layers, seed=0, dtype=torch.float32, device="cpu", **kw):
    cfg = ku.config(layers, **{k: v for k, v in kw.items() if k in ("width", "vocab", "groups", "eps", "logit_softcap")})
    sd = ku.random_weights(cfg, seed)
    path = ku.write_model(str(tmp_path / f"m{seed}"), cfg, sd)
    runner = load_runner(path, dtype, device, max_tokens=kw.get("max_tokens", 64), max_seqs=kw.get("max_seqs", 2),
                         layer_num_per_shard=kw.get("lnps"), token_budget=kw.get("token_budget", 16384))
    return cfg, sd, runner, path


def run_cut(runner, rid, toks, cuts, end=True):
    """Feed ``toks`` in portions of the sizes ``cuts`` (the rest one by one) -> logits of every position."""
    out, at = [], 0
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for i, n in enumerate(sizes):
        last = at + n == len(toks)
        r = runner.step([StepEntry(rid, toks[at:at + n], range(n))], [rid] if (last and end) else [])
        out.append(r[0][0])
        at += n
    return np.concatenate(out, 0)


HYBRID = [(ku.attn(), ku.dense()), (ku.rglru(), ku.moe()), (ku.mamba2(), None), (ku.attn(size=7, scale=2.0), ku.moe(top=1))]


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,layers", [
    ("attention", [(ku.attn(scale=2.5), None)]),
    ("attention-mha", [(ku.attn(heads=3, kv_heads=3, dim=16, vdim=16, size=5, softcap=30.0), None)]),
    ("rglru", [(ku.rglru(), None)]),
    ("rglru-one-block", [(ku.rglru(width=40, blocks=1, conv=2), None)]),
    ("mamba2", [(ku.mamba2(), None)]),
    ("mamba2-wide-state", [(ku.mamba2(heads=2, vdim=8, state=40, groups=1, norm_groups=1, conv=4), None)]),
    ("dense-ff", [(ku.rglru(conv=1), ku.dense())]),
    ("moe-ff", [(ku.rglru(), ku.moe(experts=7, top=3))]),
])
def test_mechanism_alone(tmp_path, device, name, layers):
    cfg, sd, runner, _ = build(tmp_path, layers, seed=3, device=device)
    toks = ku.tokens(45, cfg["vocab"], 1)
    got = run_cut(runner, "a", toks, [len(toks)])
    assert ku.rel_err(got, ku.oracle_logits(cfg, sd, toks)) < TOL
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_group_counts_and_caps(tmp_path, device):
    """Norm groups 1 and 4, a logit cap small enough to bend every logit, an odd width."""
    for groups, width in ((1, 44), (4, 40)):
        cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=10 + groups, device=device, groups=groups, width=width,
                                   logit_softcap=1.5)
        toks = ku.tokens(30, cfg["vocab"], 2)
        assert ku.rel_err(run_cut(runner, "a", toks, [30]), ku.oracle_logits(cfg, sd, toks)) < TOL
        runner.close()


# -------------------------------------------------- prompts, portions and decoding agree
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_portions_and_decode(tmp_path, device):
    """One request fed whole, token by token, and in portions down to two tokens (cut inside a
    chunk, at a chunk's edge, at a page's edge): every position's logits equal the oracle's."""
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=4, device=device)
    toks = ku.tokens(53, cfg["vocab"], 5)
    want = ku.oracle_logits(cfg, sd, toks)
    for cuts in ([53], [], [2, 2, 3, 13, 1, 2, 16, 9], [16, 16, 16], [20, 20], [7, 7, 7, 7, 7, 7, 7], [51]):
        assert ku.rel_err(run_cut(runner, "r", toks, cuts), want) < TOL, cuts
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_over_chunks_and_pages(tmp_path, device):
    """A short prompt, then 90 decoded tokens: they cross chunks of 20 and 7 and pages of 16, and the
    pages behind the chunk go back to the pool while the request lives."""
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=6, device=device)
    toks = ku.tokens(95, cfg["vocab"], 7)
    assert ku.rel_err(run_cut(runner, "r", toks, [5]), ku.oracle_logits(cfg, sd, toks)) < TOL
    assert runner.seq_cache.pages_trimmed > 0 and not runner.seq_cache.requests
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    """Sequences of one, two and three tokens (shorter than every convolution), alone and decoded."""
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=8, device=device)
    for n in (1, 2, 3):
        toks = ku.tokens(n, cfg["vocab"], 20 + n)
        want = ku.oracle_logits(cfg, sd, toks)
        assert ku.rel_err(run_cut(runner, "w", toks, [n]), want) < TOL
        assert ku.rel_err(run_cut(runner, "d", toks, []), want) < TOL
    runner.close()


# ------------------------------------------------------------ batches, pages and slots
@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone(tmp_path, device):
    """Requests of 1, 9, 33 and 50 tokens in one step, then decoded together while the short ones
    finish first; also cut into two micro-batches by a small token budget."""
    for budget in (16384, 40):
        cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=9, device=device, token_budget=budget)
        lens, extra = [1, 9, 33, 50], [3, 12, 0, 6]
        seqs = [ku.tokens(n + e, cfg["vocab"], 30 + i) for i, (n, e) in enumerate(zip(lens, extra))]
        want = [ku.oracle_logits(cfg, sd, s) for s in seqs]
        got = [[] for _ in seqs]
        live = [i for i in range(4)]
        res = runner.step([StepEntry(i, seqs[i][:lens[i]], range(lens[i])) for i in live], [i for i in live if extra[i] == 0])
        for i, r in zip(live, res):
            got[i].append(r[0])
        for t in range(max(extra)):
            live = [i for i in range(4) if extra[i] > t]
            res = runner.step([StepEntry(i, [seqs[i][lens[i] + t]], [0]) for i in live], [i for i in live if extra[i] == t + 1])
            for i, r in zip(live, res):
                got[i].append(r[0])
        for i in range(4):
            assert ku.rel_err(np.concatenate(got[i], 0), want[i]) < TOL, (budget, i)
        assert not runner.seq_cache.requests
        runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_used_again(tmp_path, device):
    """Requests come and go through pools of two slots and a few pages: whoever inherits a page or a
    slot (with the last owner's keys and states still in it) computes what it computes alone, and
    pools that run out grow without disturbing the live request."""
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=11, device=device, max_tokens=40, max_seqs=2)
    cache = runner.seq_cache
    a, b, c = (ku.tokens(n, cfg["vocab"], 40 + n) for n in (37, 22, 41))
    wa, wb, wc = (ku.oracle_logits(cfg, sd, s) for s in (a, b, c))
    assert ku.rel_err(run_cut(runner, "a", a, [30]), wa) < TOL
    ga = run_cut(runner, "a2", a, [10, 2], end=False)                       # stays alive
    gb = run_cut(runner, "b", b, [22])                                      # inherits a's first slot
    assert cache.slots_reused > 0 and cache.pages_reused > 0
    gc = run_cut(runner, "c", c, [3, 30])
    n0 = cache.n_slots
    others = [run_cut(runner, f"x{i}", b, [5], end=False) for i in range(3)]    # more requests than slots
    assert cache.n_slots > n0
    tail = runner.step([StepEntry("a2", [a[0]], [0])], ["a2"])[0][0]         # a2's state survived the growth
    assert ku.rel_err(tail, ku.oracle_logits(cfg, sd, a + [a[0]])[-1:]) < TOL
    for g, w in ((ga, wa), (gb, wb), (gc, wc)) + tuple((o, wb) for o in others):
        assert ku.rel_err(g, w) < TOL
    runner.close()


# ----------------------------------------------------------- keys at the edges of a chunk
@pytest.mark.parametrize("device", DEVICES)
def test_one_key_stands_out_at_chunk_edges(tmp_path, device):
    """An attention-only model whose weights are set so that one marked token's key dominates every
    query (its score is tens of units above the rest, uncapped) and its value is a large vector:
    the logits at a position tell at once whether that key was seen.  The marked token is put far
    back in the chunk, on a page border, at the chunk's first and last place, and one place
    outside; in a prompt and in decoding."""
    size, D, vocab = 24, 32, 40
    layers = [(ku.attn(heads=2, kv_heads=1, dim=16, vdim=16, size=size, scale=1.0, softcap=500.0), None)]
    cfg = ku.config(layers, width=D, vocab=vocab, groups=1)
    sd = ku.random_weights(cfg, 12, std=0.1)
    mark = 7
    e = sd["embed"].float()
    e[mark] = 0
    e[mark, :4] = 6.0                                     # the marked token's row: a few large entries
    sd["embed"] = e.to(torch.bfloat16)
    k = sd["l0.mix.k"].float()
    k[:, :4] += 3.0                                       # its key is far from the others' and aligned with ...
    q = sd["l0.mix.q"].float()
    q += k.repeat(2, 1) * 0.5                             # ... every query
    sd["l0.mix.k"], sd["l0.mix.q"] = k.to(torch.bfloat16), q.to(torch.bfloat16)
    sd["l0.mix.r1"] = torch.zeros(2).to(torch.bfloat16)   # no distance penalty to soften it
    path = ku.write_model(str(tmp_path / "edge"), cfg, sd)
    runner = load_runner(path, torch.float32, device, max_tokens=128, max_seqs=2)
    rng = np.random.default_rng(0)
    for place in (0, 15, 16, size - 1, size, 2 * size - 1, 2 * size, 2 * size + 1):
        toks = [int(t) for t in rng.integers(8, vocab, 3 * size)]
        toks[place] = mark
        want = ku.oracle_logits(cfg, sd, toks)
        seen = np.abs(want - ku.oracle_logits(cfg, sd, [t if t != mark else 9 for t in toks])).max(-1)
        lo = (place // size) * size
        assert seen[place:lo + size].min() > 50 * TOL * np.abs(want).max(), "the marked key does not stand out"
        assert ku.rel_err(run_cut(runner, "p", toks, [len(toks)]), want) < TOL, place
        assert ku.rel_err(run_cut(runner, "d", toks, [place + 1]), want) < TOL, place
    runner.close()


# ----------------------------------------------------- shards, bf16, generation, command line
@pytest.mark.parametrize("device", DEVICES)
def test_one_layer_per_shard_streams_weights(tmp_path, device):
    """layer_num_per_shard 1 without resident weights: every layer's image streams through the
    rotating weight slots each step, the state cache carries what the steps leave."""
    cfg = ku.config(HYBRID)
    sd = ku.random_weights(cfg, 13)
    path = ku.write_model(str(tmp_path / "s"), cfg, sd)
    from flexible_llm_sharding_amd.serve import load_runner as lr
    runner = lr(path, torch.float32, device, max_tokens=64, layer_num_per_shard=1, resident=False)
    toks = ku.tokens(40, cfg["vocab"], 3)
    assert ku.rel_err(run_cut(runner, "r", toks, [20, 2]), ku.oracle_logits(cfg, sd, toks)) < TOL
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_products_stay_close(tmp_path, device):
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=14, device=device, dtype=torch.bfloat16)
    toks = ku.tokens(40, cfg["vocab"], 4)
    want = ku.oracle_logits(cfg, sd, toks)
    whole, cut = run_cut(runner, "a", toks, [40]), run_cut(runner, "b", toks, [9, 2])
    assert ku.rel_err(whole, want) < 0.08 and ku.rel_err(cut, want) < 0.08
    assert ku.rel_err(cut, whole) < 0.05
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """serve.generate: prompts of unequal length, 12 new tokens each; the tokens are the oracle's
    greedy continuation (recomputed from scratch at every step)."""
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=15, device=device)
    prompts = [ku.tokens(n, cfg["vocab"], 50 + n) for n in (3, 17, 26)]
    got = generate(runner, prompts, 12)
    for p, g in zip(prompts, got):
        seq = list(p)
        for t in g:
            z = ku.oracle_logits(cfg, sd, seq)[-1]
            top2 = np.sort(z)[-2:]
            if top2[1] - top2[0] > 1e-3:              # (a tie within rounding may go either way)
                assert t == int(z.argmax())
            seq.append(t)
    assert not runner.seq_cache.requests
    runner.close()


def test_command_line_serves_a_hybrid_model(tmp_path):
    """main.py's arguments on a Kagolix checkpoint: scores [n_suffix, steps, vocab] and updated
    prompts come back in the scoring path's formats."""
    from flexible_llm_sharding_amd import api
    from flexible_llm_sharding_amd.utils.tokenizer import write_synthetic_tokenizer
    cfg = ku.config(HYBRID, vocab=64)
    sd = ku.random_weights(cfg, 16)
    path = ku.write_model(str(tmp_path / "cli"), cfg, sd)
    write_synthetic_tokenizer(path, 64)
    prompts = [("w1 w2 w3", ("w4", "w5 w6")), ("w7", ("w8 w9 w10",))]
    pk = str(tmp_path / "p.pkl")
    with open(pk, "wb") as f:
        pickle.dump(prompts, f)
    out = str(tmp_path / "o.pkl")
    api.main(["--model_path", path, "--prompt_pickle", pk, "--output_file", out, "--num_gen_token", "3",
              "--num_gpus", "0" if not gpu_available() else "1", "--dtype", "float32", "--layer_num_per_shard", "2"])
    with open(out, "rb") as f:
        scores = pickle.load(f)
    assert [s.shape for s in scores] == [(2, 3, 64), (1, 3, 64)]
    assert all(abs(float(s[i, j].astype(np.float32).sum()) - 1) < 2e-2 for s in scores for i in range(s.shape[0]) for j in range(3))
    with open(pk.replace(".pkl", "_updated.pkl"), "rb") as f:
        upd = pickle.load(f)
    assert upd[0][0] == "w1 w2 w3" and all(len(u) > len(s) for (_, us), (_, ss) in zip(upd, prompts) for u, s in zip(us, ss))


def test_trace_replay_writes_wanted_rows(tmp_path):
    """serve.replay (bin/trace_run's loop): files only for steps that want something, rows in the
    order of the entries and of ``want``."""
    from flexible_llm_sharding_amd.serve import replay
    dev = "cuda:0" if gpu_available() else "cpu"
    cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=17, device=dev)
    a, b = ku.tokens(12, cfg["vocab"], 1), ku.tokens(5, cfg["vocab"], 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [9, 0]}, {"id": "b", "tokens": b[:4], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[10:11], "want": []}, {"id": "b", "tokens": b[4:], "want": []}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[11:], "want": [0]}], "end": ["a"]}]
    said = []
    out = tmp_path / "out"
    out.mkdir()
    replay(runner, [json.dumps(s) for s in steps], str(out), said.append)
    assert said == ["done 0", "done 1", "done 2"] and sorted(p.name for p in out.iterdir()) == ["0.f32", "2.f32"]
    wa = ku.oracle_logits(cfg, sd, a)
    r0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    r2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    assert ku.rel_err(r0, wa[[9, 0]]) < TOL and ku.rel_err(r2, wa[11:]) < TOL
    runner.close()


def test_config_is_read_not_assumed(tmp_path):
    """The registry picks the family by config.json's architecture; unknown mixers and shapes that do
    not fit the config are refused at load."""
    from flexible_llm_sharding_amd.config import KagolixConfig, load_config
    cfg = ku.config(HYBRID)
    sd = ku.random_weights(cfg, 18)
    path = ku.write_model(str(tmp_path / "c"), cfg, sd)
    assert isinstance(load_config(path), KagolixConfig)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["type"] = "hyena"
    with pytest.raises(NotImplementedError):
        KagolixConfig.from_dict(bad)
    wrong = json.loads(json.dumps(cfg))
    wrong["layers"][1]["mixer"]["width"] = 96
    ku.write_model(str(tmp_path / "w"), wrong, sd)
    with pytest.raises(ValueError):
        load_runner(str(tmp_path / "w"), torch.float32, "cpu")


@pytest.mark.gpu
def test_captured_decode_steps_equal_eager(tmp_path, monkeypatch):
    """Decode steps replay as captured HIP graphs (first step of a shape eager, second captured, the
    rest replayed).  Every replay is checked against the same steps run eagerly, with eager prompt
    steps of other requests, batch-size changes and synchronisations between the replays."""
    if not gpu_available():
        pytest.skip("no GPU")

    def run(graphs: bool):
        monkeypatch.setenv("FLS_DECODE_GRAPHS", "1" if graphs else "0")
        cfg, sd, runner, _ = build(tmp_path, HYBRID, seed=21, device="cuda:0", dtype=torch.bfloat16, max_tokens=256,
                                   max_seqs=4)
        a, b, c = (ku.tokens(n, cfg["vocab"], 60 + n) for n in (40, 33, 25))
        outs = []
        runner.step([StepEntry("a", a[:10], [9]), StepEntry("b", b[:12], [11])])
        for t in range(20):
            live = [("a", a[10 + t]), ("b", b[12 + t])] + ([("c", c[9 + t - 8])] if t >= 8 else [])
            r = runner.step([StepEntry(i, [tok], [0]) for i, tok in live])
            outs += [x[0] for x in r]
            if t == 7:                                      # eager work between replays: a new prompt joins
                outs.append(runner.step([StepEntry("c", c[:9], [8])])[0][0])
            if t % 5 == 0:
                torch.cuda.synchronize()
        replays = runner._decode_graphs.replays if runner._decode_graphs is not None else 0
        runner.close()
        return np.concatenate(outs, 0), replays

    eager, n0 = run(False)
    graphed, n1 = run(True)
    assert n0 == 0 and n1 >= 12
    assert np.array_equal(eager, graphed)


def test_bench_model_builder_runs_on_cpu():
    """The benchmark's synthetic hybrid model (bench.py --hybrid) at a toy size: random layer images
    straight into a host store, a prompt step and a decode step through the runner."""
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.utils.hybrid_bench import hybrid_config, synthetic_hybrid_store
    z = dict(width=32, heads=4, kv=2, dim=8, ff=48, experts=4, top=2, eff=16, blocks=2, mh=2, mp=8, state=8, chunk=12,
             vocab=50)
    cfg = hybrid_config(z, repeats=1)
    src = synthetic_hybrid_store(cfg, "cpu", torch.float32)
    r = ShardedRunner(cfg, src, device="cpu", layer_num_per_shard=2, storage_location="cpu", compute_dtype=torch.float32,
                      state_tokens=64, state_seqs=2)
    out = r.step([StepEntry("a", list(range(20)), [19]), StepEntry("b", [1, 2, 3], [2])])
    assert out[0][0].shape == (1, 50) and np.isfinite(out[0][0]).all() and np.isfinite(out[1][0]).all()
    out = r.step([StepEntry("a", [5], [0]), StepEntry("b", [6], [])], ["a", "b"])
    assert out[1] is None and np.isfinite(out[0][0]).all() and not r.seq_cache.requests
    r.close()


def test_trace_run_program_speaks_the_protocol(tmp_path):
    """bin/trace_run as a process: steps on standard input one JSON object a line, a flushed
    'done <step>' after each, logits files for the steps that want some, exit code 0 at end of input."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = ku.config([(ku.mamba2(), ku.dense()), (ku.attn(size=6), None)], vocab=37)
    sd = ku.random_weights(cfg, 19)
    path = ku.write_model(str(tmp_path / "t"), cfg, sd)
    out = tmp_path / "logits"
    a = ku.tokens(9, 37, 4)
    p = subprocess.Popen([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "32", "--device", "cpu"], stdin=subprocess.PIPE,
                         stdout=subprocess.PIPE, text=True, cwd=root)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": a[:7], "want": [0, 6]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": a[7:8], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": a[8:], "want": [0]}], "end": ["q"]}]
    for st in steps:
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        while True:                                   # the next step only after this one's 'done'
            line = p.stdout.readline()
            assert line, "trace_run ended early"
            if line.strip() == f"done {st['step']}":
                break
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    want = ku.oracle_logits(cfg, sd, a)
    got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1),
                          np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)])
    assert not (out / "1.f32").exists() and ku.rel_err(got, want[[0, 6, 8]]) < TOL
