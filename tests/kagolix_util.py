"""Small random Kagolix models for the tests: configurations, weights on disk, and the oracle's
answers.  Sizes here are deliberately odd (3 query heads per key head, 3 norm groups, head sizes that
are not powers of two, a chunk that is no multiple of the page size) and differ from layer to layer."""
import json
import os

import numpy as np
import torch

import kagolix_oracle as oracle
from flexible_llm_sharding_amd.utils.safetensors_io import save_file


def attn(heads=6, kv_heads=2, dim=24, vdim=40, size=20, scale=0.3, softcap=8.0):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "mask": {"size": size}, "scale": scale, "softcap": softcap}}


def rglru(width=48, blocks=3, conv=4):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def mamba2(heads=4, vdim=12, state=24, groups=2, norm_groups=2, conv=3):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                        "norm_groups": norm_groups, "conv": conv}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(layers, width=48, vocab=61, groups=3, eps=1e-5, logit_softcap=12.0):
    """layers: [(mixer dict, mlp dict or None)]."""
    return {"architecture": "Kagolix", "width": width, "vocab": vocab, "norm": {"eps": eps, "groups": groups},
            "logit_softcap": logit_softcap, "layers": [dict(m, mlp=f) for m, f in layers]}


def random_weights(cfg, seed=0, std=0.35):
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def mat(*shape, s=std):
        return torch.randn(*shape, generator=g) * s

    def near_one(n):
        return 1.0 + 0.3 * torch.randn(n, generator=g)

    sd = {"embed": mat(cfg["vocab"], D, s=1.0), "head": mat(cfg["vocab"], D), "final.norm": near_one(D)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if l["mlp"] is not None else ()):
            sd[p + n] = near_one(D)
        x = p + "mix."
        if l["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd.update({x + "q": mat(H * d, D), x + "k": mat(G * d, D), x + "v": mat(G * dv, D), x + "o": mat(D, H * dv),
                       x + "q.norm": near_one(H * d), x + "k.norm": near_one(G * d),
                       x + "r1": torch.rand(H, generator=g), x + "r2": torch.rand(H, generator=g) * 2})
        elif l["type"] == "rglru":
            W, nb, taps = m["width"], m["blocks"], m["conv"]
            bw = W // nb
            sd.update({x + "y": mat(W, D), x + "y.b": mat(W), x + "x": mat(W, D), x + "x.b": mat(W),
                       x + "conv": mat(W, taps, s=0.5), x + "conv.b": mat(W), x + "ra": mat(nb, bw, bw),
                       x + "ra.b": mat(nb, bw), x + "ri": mat(nb, bw, bw), x + "ri.b": mat(nb, bw),
                       x + "lam": mat(W, s=1.0) - 2.0, x + "o": mat(D, W)})
        else:
            nh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner = nh * P
            C = inner + 2 * G * N
            sd.update({x + "in": mat(2 * inner + 2 * G * N + nh, D), x + "conv": mat(C, m["conv"], s=0.5),
                       x + "conv.b": mat(C), x + "dt_bias": mat(nh, s=1.0), x + "A_log": mat(nh, s=0.7),
                       x + "D": mat(nh, s=1.0), x + "norm": near_one(inner), x + "o": mat(D, inner)})
        if l["mlp"] is not None:
            y = p + "mlp."
            if l["mlp"]["kind"] == "dense":
                ff = l["mlp"]["ff"]
                sd.update({y + "up": mat(ff, D), y + "down": mat(D, ff), y + "act": mat(2, s=1.0)})
            else:
                E, ff = l["mlp"]["router"]["experts"], l["mlp"]["expert"]["ff"]
                sd.update({y + "router": mat(E, D, s=1.0), y + "correction": mat(E, s=0.2)})
                for e in range(E):
                    sd.update({f"{y}e{e}.gate": mat(ff, D), f"{y}e{e}.up": mat(ff, D), f"{y}e{e}.down": mat(D, ff)})
    return {k: v.to(torch.bfloat16) for k, v in sd.items()}


def write_model(path, cfg, sd):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(sd, os.path.join(path, "model.safetensors"))
    return path


def oracle_logits(cfg, sd, tokens):
    return oracle.forward(cfg, sd, list(tokens)).numpy()


def rel_err(got, want):
    """Mean-free RMS difference of logit rows over the RMS of the wanted rows (the worst row)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / (np.sqrt((w ** 2).mean(-1)) + 1e-12)).max())


def tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()
