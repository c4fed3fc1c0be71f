"""Step-by-step serving of a stateful (hybrid) model: loading, trace replay and greedy generation.

The scoring entry point (``api.run_rank``) hands a hybrid model's prompts to :func:`generate`;
``bin/trace_run`` replays a recorded sequence of steps with :func:`replay`.  Both drive
:meth:`~.engine.ShardedRunner.step`: the same shard schedule, weight slots, sequence state cache and
kernels.
"""
from __future__ import annotations

import json
import os
import sys
from typing import List, Optional, Sequence

import numpy as np
import torch

from .config import is_hybrid, load_config, resolve_dtype
from .engine import ShardedRunner
from .runtime.batch import StepEntry
from .runtime.weights import CheckpointSource, HostStore


def ensure_built(device: torch.device) -> None:
    """Build what serving a hybrid model on a GPU loads, if it is not there: the host runtime (pinned
    memory) and the stateful-model kernels.  Nothing of the scoring kernels is compiled."""
    if device.type != "cuda":
        return
    from ._native import build
    build.build_runtime()
    build.build_seq_kernels()


def load_runner(model_path: str, dtype: torch.dtype, device=None, max_tokens: int = 4096, max_seqs: int = 8,
                layer_num_per_shard: Optional[int] = None, resident: bool = True, token_budget: int = 16384,
                storage_location: str = "cpu") -> ShardedRunner:
    """A runner for the hybrid model in ``model_path`` (config.json + model.safetensors).  ``dtype``:
    the element type of the matrix products, bf16 or fp32; everything else is fp32 either way."""
    cfg = load_config(model_path)
    if not is_hybrid(cfg):
        raise NotImplementedError("step-by-step serving needs a hybrid architecture (config.json \"architecture\")")
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("hybrid models run with bfloat16 or float32 matrix products")
    dev = torch.device(device if device is not None else ("cuda:0" if torch.cuda.is_available() else "cpu"))
    ensure_built(dev)
    src = HostStore.from_source(CheckpointSource(cfg, model_path, dtype), pinned=dev.type == "cuda")
    lnps = layer_num_per_shard or len(cfg.layer_names())
    return ShardedRunner(cfg, src, device=dev, layer_num_per_shard=lnps, storage_location=storage_location,
                         resident=resident, token_budget=token_budget, compute_dtype=dtype,
                         state_tokens=max_tokens, state_seqs=max_seqs)


def replay(runner: ShardedRunner, lines, out_dir: str, say=None) -> int:
    """Run recorded steps, one JSON object a line: {"step": n, "entries": [{"id", "tokens", "want"}],
    "end": [ids]}.  The logits of a step's wanted places go to ``out_dir/<n>.f32`` ([wanted, vocab]
    little-endian fp32, in the order of the entries and of ``want``); ``say("done <n>")`` after every
    step."""
    n_steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [StepEntry(e["id"], e["tokens"], e.get("want") or ()) for e in st.get("entries", [])]
        outs = runner.step(entries, st.get("end") or ())
        rows = [o[0] for o in outs if o is not None]
        if rows:
            a = np.ascontiguousarray(np.concatenate(rows, 0), dtype="<f4")
            tmp = os.path.join(out_dir, f".{st['step']}.f32.part")
            with open(tmp, "wb") as f:
                f.write(a.tobytes())
            os.replace(tmp, os.path.join(out_dir, f"{st['step']}.f32"))
        if say is not None:
            say(f"done {st['step']}")
        n_steps += 1
    return n_steps


def generate(runner: ShardedRunner, prompts: Sequence[Sequence[int]], num_new: int, stop_ids: Sequence[int] = (),
             want_probs: bool = False):
    """Greedy generation through the runner's scheduler: one step for all prompts (different lengths,
    packed without padding), then one token per live request and step; a request that emits a stop id
    leaves the batch and its state is given back.  -> (tokens per prompt, and with ``want_probs`` per
    prompt a [steps, vocab] fp16 array of next-token probabilities)."""
    n = len(prompts)
    out: List[List[int]] = [[] for _ in range(n)]
    probs: List[list] = [[] for _ in range(n)]
    live = list(range(n))
    feed = {i: list(prompts[i]) for i in live}
    stop = set(int(s) for s in stop_ids)
    for it in range(num_new):
        if not live:
            break
        last = it == num_new - 1
        entries = [StepEntry(("gen", i), feed[i], [len(feed[i]) - 1]) for i in live]
        ends = [("gen", i) for i in live] if last else []
        res = runner.step(entries, ends)
        nxt = []
        for i, r in zip(live, res):
            logits, am = r
            t = int(am[0])
            out[i].append(t)
            if want_probs:
                z = torch.from_numpy(np.array(logits[0], dtype=np.float32))
                probs[i].append(torch.softmax(z, -1).to(torch.float16).numpy())
            if t in stop and not last:
                runner.seq_cache.release(("gen", i))
            else:
                nxt.append(i)
                feed[i] = [t]
        live = nxt
    if want_probs:
        return out, [np.stack(p) if p else np.zeros((0, runner.cfg.vocab_size), np.float16) for p in probs]
    return out


def run_prompts(args, cfg, tok, prompts):
    """``main.py`` semantics for a hybrid model: every (prefix, suffixes) prompt is scored at the end
    of each suffix and extended greedily by ``--num_gen_token`` tokens; prefix + suffix is one request
    (a recurrent state cannot be shared between suffixes the way prefix K/V can).
    -> (scores per prompt [n_suffix, num_gen_token, vocab] fp16, updated prompts)."""
    from .utils.tokenizer import tokenize_prompts
    dtype = resolve_dtype(getattr(args, "dtype", None) or "bfloat16")
    if dtype == torch.float16:
        dtype = torch.bfloat16
    tps = tokenize_prompts(tok, prompts, getattr(args, "max_token_len", None) or 4096)
    reqs, owner = [], []
    for pi, tp in enumerate(tps):
        for si, s in enumerate(tp.suffixes):
            reqs.append(list(tp.prefix) + list(s))
            owner.append((pi, si))
    device = None if torch.cuda.is_available() else "cpu"
    runner = load_runner(args.model_path, dtype, device, max_tokens=sum(len(r) for r in reqs) + len(reqs) * args.num_gen_token,
                         max_seqs=max(1, len(reqs)), layer_num_per_shard=args.layer_num_per_shard,
                         resident=bool(getattr(args, "resident", False)),
                         token_budget=getattr(args, "token_budget", None) or 16384,
                         storage_location=args.storage_location)
    try:
        toks, probs = generate(runner, reqs, args.num_gen_token, want_probs=True)
    finally:
        stats = dict(runner.stats)
        runner.close()
    scores = [np.zeros((len(tp.suffixes), args.num_gen_token, cfg.vocab_size), np.float16) for tp in tps]
    updated = [(p, list(s)) for p, s in prompts]
    for (pi, si), t, pr in zip(owner, toks, probs):
        scores[pi][si, :pr.shape[0]] = pr
        updated[pi][1][si] = updated[pi][1][si] + tok.decode(t)
    return scores, [(p, tuple(s)) for p, s in updated], stats


def trace_main(argv=None) -> int:
    """bin/trace_run: --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N; steps on stdin."""
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description="Replay recorded serving steps and write logits.")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, default=4096, help="most tokens live requests hold at once")
    ap.add_argument("--device", default=None)
    ap.add_argument("--layer-num-per-shard", type=int, default=None)
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    runner = load_runner(a.model, resolve_dtype(a.dtype), a.device, max_tokens=a.max_tokens,
                         layer_num_per_shard=a.layer_num_per_shard)

    def say(text: str) -> None:
        sys.stdout.write(text + "\n")
        sys.stdout.flush()
    try:
        replay(runner, sys.stdin, a.out, say)
    finally:
        runner.close()
    return 0
