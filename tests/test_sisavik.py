"""Sisavik through the framework (config registry, weight images, sequence state cache, step
scheduler, kernels) against the plain float64 oracle in ``sisavik_oracle.py``.

Every test runs on the CPU backend (plain PyTorch ops) and, marked ``gpu``, on the HIP kernels.  The
models are tiny and random; fp32 matrix products make the comparison sharp (a window one token off,
a lost state, a forgotten kept token or a wrong page shows as an error thousands of times the
tolerance), and one test runs the bf16 mode.  Where random weights would hide a fault, the weights
are set so that one key dominates."""
import json
import os
import pickle
import subprocess
import sys

import numpy as np
import pytest
import torch

import sisavik_oracle as oracle
import sisavik_util as su
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
    cfg, ranks = su.config(layers, **{k: v for k, v in kw.items() if k in ("width", "vocab", "eps", "taps")})
    sd = su.random_weights(cfg, ranks, seed, **({"std": kw["std"]} if "std" in kw else {}))
    path = su.write_model(str(tmp_path / f"m{seed}"), cfg, sd)
    runner = load_runner(path, dtype, device, max_tokens=kw.get("max_tokens", 64), max_seqs=kw.get("max_seqs", 2),
                         layer_num_per_shard=kw.get("lnps"), token_budget=kw.get("token_budget", 16384))
    return cfg, sd, runner, path


def run_cut(runner, rid, toks, cuts, end=True):
    """Feed ``toks`` in portions of the sizes ``cuts`` (the rest one by one) -> logits of every position."""
    out, at = [], 0
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        last = at + n == len(toks)
        r = runner.step([StepEntry(rid, toks[at:at + n], range(n))], [rid] if (last and end) else [])
        out.append(r[0][0])
        at += n
    return np.concatenate(out, 0)


# own latent, a parallel pair, a second own latent, and two layers that read the third layer's latent
STACK = [(su.latent(), su.dense()), (su.parallel(), su.dense(ff=28)), (su.latent(heads=2, dim=8, rot_dim=4, vdim=16, size=13), None),
         (su.latent(heads=4, dim=6, rot_dim=4, vdim=5, kv_rank=14, size=5, kv_from=2), su.dense()),
         (su.parallel(heads=4, kv_heads=4, dim=10, rot_dims=10, size=11, keep_first=0, rheads=3, rdim=7), None)]


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,layers,kw", [
    ("latent", [(su.latent(scale=1.5), None)], {}),
    ("latent-one-head-window-1", [(su.latent(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5, q_rank=4, size=1), None)], {}),
    ("latent-shared", [(su.latent(), None), (su.latent(heads=2, dim=5, vdim=7, size=4, kv_from=0), None)], {}),
    ("sigmoid-attention", [(su.parallel(right_scale=0.0, scale=1.2), None)], {}),
    ("sigmoid-attention-mha-full-rotation", [(su.parallel(heads=3, kv_heads=3, dim=8, rot_dims=8, keep_first=0, right_scale=0.0), None)], {}),
    ("delta-rule", [(su.parallel(left_scale=0.0), None)], {}),
    ("delta-rule-head-33", [(su.parallel(left_scale=0.0, rheads=1, rdim=33, decay_rank=1), None)], {}),
    ("delta-rule-head-64", [(su.parallel(left_scale=0.0, rheads=2, rdim=64), None)], {"width": 24}),
    ("delta-rule-head-128", [(su.parallel(left_scale=0.0, rheads=1, rdim=128), None)], {"width": 24}),
    ("no-input-conv", [(su.latent(), su.dense()), (su.parallel(), su.dense())], {"taps": 1}),
    ("five-taps", [(su.latent(), su.dense()), (su.parallel(), su.dense())], {"taps": 5}),
    ("feed-forward", [(su.latent(size=2), su.dense(ff=100))], {}),
])
def test_mechanism_alone(tmp_path, device, name, layers, kw):
    cfg, sd, runner, _ = build(tmp_path, layers, seed=3, device=device, **kw)
    toks = su.tokens(45, cfg["vocab"], 1)
    want = su.oracle_logits(cfg, sd, toks)
    assert su.rel_err(run_cut(runner, "a", toks, [len(toks)]), want) < TOL
    assert su.rel_err(run_cut(runner, "b", toks, [30, 2]), want) < TOL
    runner.close()


def test_oracle_parts_agree_with_their_definitions():
    """The oracle's own pieces on hand-made inputs: the window, the rotation of a pair, the input
    convolution's tap order, one step of the delta rule."""
    assert [j for j in range(12) if oracle.sees(10, j, 3, 2)] == [0, 1, 8, 9, 10] and not oracle.sees(3, 4, 9)
    x = torch.tensor([[[1.0, 0.0, 5.0, 6.0]]], dtype=torch.float64)
    r = oracle.rotate(x, torch.tensor([3]), 2, 100.0)
    assert torch.allclose(r[0, 0], torch.tensor([np.cos(3.0), np.sin(3.0), 5.0, 6.0], dtype=torch.float64))
    h = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    w = torch.tensor([[0.5, 0.25, 2.0]], dtype=torch.float64)          # taps 3: w[:, 2] weighs the current row
    assert torch.allclose(oracle.input_conv(h, w)[:, 0], torch.tensor([1 + 2.0, 10 + 20 + 0.25, 100 + 200 + 2.5 + 0.5], dtype=torch.float64))


# ----------------------------------------------- prompts, portions, decoding, first tokens
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_portions_and_decode(tmp_path, device):
    """The same sequence whole, token by token, and in portions of 2, 3, 7, 16 and 17 tokens: windows,
    kept tokens, convolution history and recurrent state all cross the cuts."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=5, device=device)
    toks = su.tokens(50, cfg["vocab"], 2)
    want = su.oracle_logits(cfg, sd, toks)
    for cuts in ([50], [], [2, 2, 3, 7, 16, 17], [17, 16, 2], [1, 2, 40]):
        assert su.rel_err(run_cut(runner, "r", toks, cuts), want) < TOL, cuts
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_over_windows_and_pages(tmp_path, device):
    """A short prompt, then 120 decoded tokens: every window passes over decoded tokens, pages of 16
    fill and the pages behind all windows go back to the pool while the request lives -- except the
    page of the first tokens, which the parallel layer keeps."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=6, device=device)
    toks = su.tokens(125, cfg["vocab"], 7)
    got = run_cut(runner, "r", toks, [5], end=False)
    assert su.rel_err(got, su.oracle_logits(cfg, sd, toks)) < TOL
    cache = runner.seq_cache
    req = cache.requests["r"]
    assert cache.pages_trimmed > 0 and req.pages[0] >= 0 and req.pages[1] < 0
    cache.release("r")
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    """Sequences of one, two and three tokens (shorter than the convolution, the windows and the kept
    tokens), alone and decoded."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=8, device=device, taps=4)
    for n in (1, 2, 3):
        toks = su.tokens(n, cfg["vocab"], 20 + n)
        want = su.oracle_logits(cfg, sd, toks)
        assert su.rel_err(run_cut(runner, "w", toks, [n]), want) < TOL
        assert su.rel_err(run_cut(runner, "d", toks, []), want) < TOL
    runner.close()


# ------------------------------------------------------------ batches, pages and slots
@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone(tmp_path, device):
    """Requests of 1, 9, 33 and 50 tokens in one step, then decoded together while the short ones
    finish first; also cut into two micro-batches by a small token budget."""
    for budget in (16384, 40):
        cfg, sd, runner, _ = build(tmp_path, STACK, seed=9, device=device, token_budget=budget)
        lens, extra = [1, 9, 33, 50], [3, 12, 0, 6]
        seqs = [su.tokens(n + e, cfg["vocab"], 30 + i) for i, (n, e) in enumerate(zip(lens, extra))]
        want = [su.oracle_logits(cfg, sd, s) for s in seqs]
        got = [[] for _ in seqs]
        live = list(range(4))
        res = runner.step([StepEntry(i, seqs[i][:lens[i]], range(lens[i])) for i in live], [i for i in live if extra[i] == 0])
        for i, r in zip(live, res):
            got[i].append(r[0])
        for t in range(max(extra)):
            live = [i for i in range(4) if extra[i] > t]
            res = runner.step([StepEntry(i, [seqs[i][lens[i] + t]], [0]) for i in live], [i for i in live if extra[i] == t + 1])
            for i, r in zip(live, res):
                got[i].append(r[0])
        for i in range(4):
            assert su.rel_err(np.concatenate(got[i], 0), want[i]) < TOL, (budget, i)
        assert not runner.seq_cache.requests
        runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_used_again(tmp_path, device):
    """Requests come and go through pools of two slots and a few pages: whoever inherits a page or a
    slot (with the last owner's latent rows, keys, convolution inputs and states still in it) computes
    what it computes alone, and pools that run out grow without disturbing the live request."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=11, device=device, max_tokens=40, max_seqs=2)
    cache = runner.seq_cache
    a, b, c = (su.tokens(n, cfg["vocab"], 40 + n) for n in (37, 22, 41))
    wa, wb, wc = (su.oracle_logits(cfg, sd, s) for s in (a, b, c))
    assert su.rel_err(run_cut(runner, "a", a, [30]), wa) < TOL
    ga = run_cut(runner, "a2", a, [10, 2], end=False)                       # stays alive
    gb = run_cut(runner, "b", b, [22])                                      # inherits a's first slot
    assert cache.slots_reused > 0 and cache.pages_reused > 0
    gc = run_cut(runner, "c", c, [3, 30])
    n0 = cache.n_slots
    others = [run_cut(runner, f"x{i}", b, [5], end=False) for i in range(3)]    # more requests than slots
    assert cache.n_slots > n0
    tail = runner.step([StepEntry("a2", [a[0]], [0])], ["a2"])[0][0]         # a2's state survived the growth
    assert su.rel_err(tail, su.oracle_logits(cfg, sd, a + [a[0]])[-1:]) < TOL
    for g, w in ((ga, wa), (gb, wb), (gc, wc)) + tuple((o, wb) for o in others):
        assert su.rel_err(g, w) < TOL
    runner.close()


# ------------------------------------------- one key that stands out, at every kind of edge
def _marked_latent_model(tmp_path, size):
    """One latent attention layer whose weights make the marked token's key dominate every query: its
    embedding is a few large entries, W_dkv maps them to a latent far from the others', and the
    unrotated queries are aligned with W_uk of that latent (the rotated part stays small)."""
    D, vocab, mark = 32, 40, 7
    layers = [(su.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8, q_rank=12, size=size, scale=3.0), None)]
    cfg, ranks = su.config(layers, width=D, vocab=vocab, taps=1)
    sd = {k: v.float() for k, v in su.random_weights(cfg, ranks, 12, std=0.1).items()}
    sd["embed"][mark] = 0
    sd["embed"][mark, :4] = 6.0
    sd["l0.mix.dkv"][:8, :4] += 2.0                        # the marked token's latent: all entries large and alike
    sd["l0.mix.dkv.norm"][:] = 1.0
    sd["l0.mix.uk"][:] = 0.05 * sd["l0.mix.uk"] + 0.5      # every head's key ~ sum of the latent: large for the mark
    sd["l0.mix.uq"].view(2, 12, 12)[:, :8, :] += 0.6       # unrotated queries: positive sums for every token
    sd["l0.mix.dq"][:] = sd["l0.mix.dq"].abs()
    sd["embed"][:] = sd["embed"].abs()
    sd["embed"][:, :4] = 0.0                                # only the marked token excites the large latent
    sd["embed"][mark, :4] = 6.0
    sd["l0.mix.uv"][:] *= 8.0
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    return cfg, sd, su.write_model(str(tmp_path / "edge_l"), cfg, sd), mark, vocab


@pytest.mark.parametrize("device", DEVICES)
def test_one_key_stands_out_at_window_edges_latent(tmp_path, device):
    """The marked token far back, on a page border, at the window's last and first place and one place
    outside, seen from a prompt position and from a decoded one."""
    size = 21
    cfg, sd, path, mark, vocab = _marked_latent_model(tmp_path, size)
    runner = load_runner(path, torch.float32, device, max_tokens=128, max_seqs=2)
    rng = np.random.default_rng(0)
    n = 70
    for place in (0, 15, 16, 31, 32, n - size - 1, n - size, n - size + 1, n - 2):
        toks = [int(t) for t in rng.integers(8, vocab, n)]
        toks[place] = mark
        want = su.oracle_logits(cfg, sd, toks)
        seen = np.abs(want - su.oracle_logits(cfg, sd, [t if t != mark else 9 for t in toks])).max(-1)
        inside = [i for i in range(place + 1, n) if i - place < size]
        outside = [i for i in range(place + size, n)]
        assert not inside or seen[inside].min() > 50 * TOL * np.abs(want).max(), "the marked key does not stand out"
        assert not outside or seen[outside].max() == 0.0
        assert su.rel_err(run_cut(runner, "p", toks, [n]), want) < TOL, place
        assert su.rel_err(run_cut(runner, "d", toks, [place + 1]), want) < TOL, place
        assert su.rel_err(run_cut(runner, "e", toks, [min(n, place + size - 1)]), want) < TOL, place
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_kept_first_tokens_and_window_edges_sigmoid(tmp_path, device):
    """The left mixer alone, values scaled up: every visible key adds sigmoid(score + b) times a large
    value with no normalisation, so one key too many or too few moves the output.  The marked token
    sits inside the kept first tokens, just past them, at the window's two edges and far back, in
    sequences long enough that the kept tokens lie hundreds of positions (and many pages) behind."""
    size, keep, D, vocab, mark = 19, 5, 24, 40, 7
    layers = [(su.parallel(heads=4, kv_heads=2, dim=8, rot_dims=4, size=size, keep_first=keep, scale=0.3, right_scale=0.0,
                           rheads=1, rdim=4, decay_rank=2), None)]
    cfg, ranks = su.config(layers, width=D, vocab=vocab, taps=1)        # (no input convolution: a token stays in its place)
    sd = {k: v.float() for k, v in su.random_weights(cfg, ranks, 13, std=0.2).items()}
    sd["embed"][mark] *= 6.0                               # its key (= its value) is several times the others'
    sd["l0.mix.left.pb"][:] = 0.5
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    path = su.write_model(str(tmp_path / "edge_s"), cfg, sd)
    runner = load_runner(path, torch.float32, device, max_tokens=512, max_seqs=2)
    rng = np.random.default_rng(1)
    n = 300
    for place in (0, keep - 1, keep, 16, n - size - 1, n - size, n - size + 1, n - 1):
        toks = [int(t) for t in rng.integers(8, vocab, n)]
        toks[place] = mark
        want = su.oracle_logits(cfg, sd, toks)
        seen = np.abs(want - su.oracle_logits(cfg, sd, [t if t != mark else 9 for t in toks])).max(-1)
        last_seen = seen[n - 1] > 50 * TOL * np.abs(want).max()
        assert last_seen == (place < keep or n - 1 - place < size), place
        assert su.rel_err(run_cut(runner, "p", toks, [n])[-40:], want[-40:]) < TOL, place
        got = run_cut(runner, "d", toks, [n - 25])
        assert su.rel_err(got[-40:], want[-40:]) < TOL, place
    assert runner.seq_cache.pages_trimmed > 0
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_remembers_a_far_token(tmp_path, device):
    """The right mixer alone with a decay close to 1: a token hundreds of positions back still shapes
    the state, through a prompt cut into portions and through decoding."""
    layers = [(su.parallel(left_scale=0.0, rheads=2, rdim=12, decay_rank=3), None)]
    cfg, ranks = su.config(layers, width=20, vocab=30, taps=2)
    sd = {k: v.float() for k, v in su.random_weights(cfg, ranks, 14).items()}
    sd["l0.mix.right.w0"][:] = -9.0                        # w = exp(-0.6 sigmoid(-9 + small)) ~ 1 - 7e-5
    sd["l0.mix.right.w2"][:] *= 0.05
    sd["l0.mix.right.a.b"][:] = -6.0                       # little is removed
    sd["l0.mix.right.a"][:] *= 0.1
    sd["embed"][29] *= 5.0                                 # the far token writes a large k v^T into the state
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    path = su.write_model(str(tmp_path / "far"), cfg, sd)
    runner = load_runner(path, torch.float32, device, max_tokens=512, max_seqs=2)
    toks = [29] + su.tokens(259, 28, 5)
    want = su.oracle_logits(cfg, sd, toks)
    other = su.oracle_logits(cfg, sd, [28] + toks[1:])
    assert su.rel_err(other[-1:], want[-1:]) > 50 * TOL, "the first token no longer matters at the end"
    assert su.rel_err(run_cut(runner, "a", toks, [100, 2, 130]), want) < 2 * TOL
    runner.close()


# ----------------------------------------------------- shards, bf16, generation, command line
@pytest.mark.parametrize("device", DEVICES)
def test_one_layer_per_shard_streams_weights(tmp_path, device):
    cfg, ranks = su.config(STACK)
    sd = su.random_weights(cfg, ranks, 13)
    path = su.write_model(str(tmp_path / "s"), cfg, sd)
    runner = load_runner(path, torch.float32, device, max_tokens=64, layer_num_per_shard=1, resident=False)
    toks = su.tokens(40, cfg["vocab"], 3)
    assert su.rel_err(run_cut(runner, "r", toks, [20, 2]), su.oracle_logits(cfg, sd, toks)) < TOL
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_products_stay_close(tmp_path, device):
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=14, device=device, dtype=torch.bfloat16)
    toks = su.tokens(40, cfg["vocab"], 4)
    want = su.oracle_logits(cfg, sd, toks)
    whole, cut = run_cut(runner, "a", toks, [40]), run_cut(runner, "b", toks, [9, 2])
    assert su.rel_err(whole, want) < 0.08 and su.rel_err(cut, want) < 0.08
    assert su.rel_err(cut, whole) < 0.05
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """serve.generate: prompts of unequal length, 12 new tokens each; the tokens are the oracle's
    greedy continuation (recomputed from scratch at every step)."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=15, device=device)
    prompts = [su.tokens(n, cfg["vocab"], 50 + n) for n in (3, 17, 26)]
    got = generate(runner, prompts, 12)
    for p, g in zip(prompts, got):
        seq = list(p)
        for t in g:
            z = su.oracle_logits(cfg, sd, seq)[-1]
            top2 = np.sort(z)[-2:]
            if top2[1] - top2[0] > 1e-3:              # (a tie within rounding may go either way)
                assert t == int(z.argmax())
            seq.append(t)
    assert not runner.seq_cache.requests
    runner.close()


def test_command_line_serves_the_model(tmp_path):
    from flexible_llm_sharding_amd import api
    from flexible_llm_sharding_amd.utils.tokenizer import write_synthetic_tokenizer
    cfg, ranks = su.config(STACK, vocab=64)
    sd = su.random_weights(cfg, ranks, 16)
    path = su.write_model(str(tmp_path / "cli"), cfg, sd)
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


def test_config_is_read_not_assumed(tmp_path):
    """The registry picks the family by config.json's architecture; the decay map's rank comes from the
    checkpoint; layers that contradict each other or the checkpoint are refused at load."""
    from flexible_llm_sharding_amd.config import SisavikConfig, load_config
    cfg, ranks = su.config(STACK)
    sd = su.random_weights(cfg, ranks, 18)
    path = su.write_model(str(tmp_path / "c"), cfg, sd)
    c = load_config(path)
    assert isinstance(c, SisavikConfig) and c.layers[1].mixer["right"]["decay_rank"] == 5 and c.kv_owner(3) == 2
    for edit in (lambda d: d["layers"][0].update(type="hyena"),
                 lambda d: d["layers"][3]["mixer"].update(kv_rank=15),
                 lambda d: d["layers"][3]["mixer"].update(kv_from=1),
                 lambda d: d["layers"][1]["mixer"]["left"].update(vdim=8)):
        bad = json.loads(json.dumps(cfg))
        edit(bad)
        with pytest.raises((NotImplementedError, ValueError)):
            SisavikConfig.from_dict(bad, path)
    wrong = json.loads(json.dumps(cfg))
    wrong["layers"][0]["mixer"]["q_rank"] = 20
    su.write_model(str(tmp_path / "w"), wrong, sd)
    with pytest.raises(ValueError):
        load_runner(str(tmp_path / "w"), torch.float32, "cpu")


@pytest.mark.gpu
def test_captured_decode_steps_equal_eager(tmp_path, monkeypatch):
    """Decode steps replay as captured HIP graphs; every replay is checked against the same steps run
    eagerly, with eager prompt steps of other requests and batch-size changes between the replays."""
    if not gpu_available():
        pytest.skip("no GPU")

    def run(graphs: bool):
        monkeypatch.setenv("FLS_DECODE_GRAPHS", "1" if graphs else "0")
        cfg, sd, runner, _ = build(tmp_path, STACK, seed=21, device="cuda:0", dtype=torch.bfloat16, max_tokens=256, max_seqs=4)
        a, b, c = (su.tokens(n, cfg["vocab"], 60 + n) for n in (40, 33, 25))
        outs = []
        runner.step([StepEntry("a", a[:10], [9]), StepEntry("b", b[:12], [11])])
        for t in range(20):
            live = [("a", a[10 + t]), ("b", b[12 + t])] + ([("c", c[9 + t - 8])] if t >= 8 else [])
            r = runner.step([StepEntry(i, [tok], [0]) for i, tok in live])
            outs += [x[0] for x in r]
            if t == 7:
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


def test_trace_run_program_replays_steps(tmp_path):
    """bin/trace_run as a process on a two-request schedule: prompts of unequal length in one step,
    then one token each; a flushed 'done <step>' after each step, logits files for the steps that
    want some, exit code 0 at end of input."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg, ranks = su.config(STACK[:4], vocab=37)
    sd = su.random_weights(cfg, ranks, 19)
    path = su.write_model(str(tmp_path / "t"), cfg, sd)
    out = tmp_path / "logits"
    a, b = su.tokens(9, 37, 4), su.tokens(3, 37, 5)
    p = subprocess.Popen([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "32", "--device", "cpu"], stdin=subprocess.PIPE,
                         stdout=subprocess.PIPE, text=True, cwd=root)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": a[:7], "want": [0, 6]}, {"id": "s", "tokens": b[:1], "want": [0]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": a[7:8], "want": []}, {"id": "s", "tokens": b[1:2], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": a[8:], "want": [0]}, {"id": "s", "tokens": b[2:], "want": [0]}], "end": ["q", "s"]}]
    for st in steps:
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        while True:
            line = p.stdout.readline()
            assert line, "trace_run ended early"
            if line.strip() == f"done {st['step']}":
                break
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    wa, wb = su.oracle_logits(cfg, sd, a), su.oracle_logits(cfg, sd, b)
    got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(3, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)])
    assert not (out / "1.f32").exists()
    assert su.rel_err(got, np.concatenate([wa[[0, 6]], wb[[0]], wa[[8]], wb[[2]]])) < TOL


def test_bench_model_builder_runs_on_cpu():
    """The benchmark's synthetic stacks (bench.py --hybrid --hybrid-family sisavik) at a toy size: random
    layer images straight into a host store, a prompt step and a decode step through the runner."""
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.utils.hybrid_bench import kagolix_dense_config, sisavik_config, synthetic_hybrid_store
    z = dict(width=64, heads=4, kv=2, dim=16, ff=96, experts=4, top=2, eff=16, blocks=2, mh=2, mp=8, state=8, chunk=12, vocab=50)
    for cfg in (sisavik_config(z, repeats=1), kagolix_dense_config(z, repeats=1)):
        src = synthetic_hybrid_store(cfg, "cpu", torch.float32)
        r = ShardedRunner(cfg, src, device="cpu", layer_num_per_shard=2, storage_location="cpu", compute_dtype=torch.float32,
                          state_tokens=64, state_seqs=2)
        out = r.step([StepEntry("a", list(range(20)), [19]), StepEntry("b", [1, 2, 3], [2])])
        assert out[0][0].shape == (1, 50) and np.isfinite(out[0][0]).all() and np.isfinite(out[1][0]).all()
        out = r.step([StepEntry("a", [5], [0]), StepEntry("b", [6], [])], ["a", "b"])
        assert out[1] is None and np.isfinite(out[0][0]).all() and not r.seq_cache.requests
        r.close()


@pytest.mark.parametrize("device", DEVICES)
def test_head_sizes_of_the_matrix_core_kernels(tmp_path, device):
    """bf16 with head sizes that the matrix-core kernels serve on the GPU: prompts unfold the latent
    into per-head keys of 128 and values of 64, decode steps fold it (key rows of 192, 128 value
    columns: the heads of a token share one tile), the sigmoid attention has heads of 64; a prompt of
    several row tiles, then decoding past the windows.  Whole-prompt and decoded logits both stay
    within bf16 rounding of the oracle, and of each other."""
    layers = [(su.latent(heads=3, dim=64, rot_dim=64, vdim=64, kv_rank=128, q_rank=20, size=150, scale=0.12), su.dense()),
              (su.parallel(heads=4, kv_heads=2, dim=64, rot_dims=32, size=40, keep_first=5, scale=0.15, rheads=2, rdim=64), None),
              (su.latent(heads=2, dim=64, rot_dim=64, vdim=128, kv_rank=128, q_rank=12, size=33, scale=0.12, kv_from=0), None)]
    cfg, sd, runner, _ = build(tmp_path, layers, seed=23, device=device, dtype=torch.bfloat16, max_tokens=512, std=0.2)
    toks = su.tokens(230, cfg["vocab"], 6)
    want = su.oracle_logits(cfg, sd, toks)
    whole = run_cut(runner, "a", toks, [230])
    cut = run_cut(runner, "b", toks, [190])
    assert su.rel_err(whole, want) < 0.08 and su.rel_err(cut, want) < 0.08
    assert su.rel_err(cut, whole) < 0.06
    runner.close()
