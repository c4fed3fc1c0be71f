"""Small random Sisavik models for the tests: configurations, weights on disk, and the oracle's
answers.  Sizes are deliberately odd and unlike each other (3 query heads per key head, head sizes
that are no powers of two, windows that are no multiples of the page size, a rotation over part of a
head, left and right scales far from 1) and differ from layer to layer."""
import json
import os

import numpy as np
import torch

import sisavik_oracle as oracle
from flexible_llm_sharding_amd.utils.safetensors_io import save_file


def latent(heads=3, dim=12, rot_dim=6, vdim=10, kv_rank=14, q_rank=18, size=9, scale=0.4, base=50.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "mask": {"size": size}, "rot": {"dims": rot_dim, "base": base}, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def parallel(heads=6, kv_heads=2, dim=12, rot_dims=8, size=7, keep_first=3, scale=0.5, base=300.0, rheads=2, rdim=10,
             left_scale=0.7, right_scale=1.3, decay_rank=5):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": size, "keep_first": keep_first},
                 "rot": {"dims": rot_dims, "base": base}, "scale": scale},
        "right": {"heads": rheads, "dim": rdim}, "left_scale": left_scale, "right_scale": right_scale},
        "decay_rank": decay_rank}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def config(layers, width=36, vocab=53, eps=1e-5, taps=3):
    """layers: [(mixer dict, mlp dict or None)] -> (config.json's content, the rank of each layer's decay map)."""
    ls, ranks = [], {}
    for i, (m, f) in enumerate(layers):
        m = json.loads(json.dumps(m))
        if "decay_rank" in m:
            ranks[i] = m.pop("decay_rank")
        ls.append(dict(m, mlp=f))
    return {"architecture": "Sisavik", "width": width, "vocab": vocab, "norm": {"eps": eps}, "canon": {"taps": taps},
            "layers": ls}, ranks


def random_weights(cfg, ranks, seed=0, std=0.3):
    g = torch.Generator().manual_seed(seed)
    D, taps = cfg["width"], cfg["canon"]["taps"]

    def mat(*shape, s=std):
        return torch.randn(*shape, generator=g) * s

    def near_one(n):
        return 1.0 + 0.3 * torch.randn(n, generator=g)

    sd = {"embed": mat(cfg["vocab"], D, s=1.0), "head": mat(cfg["vocab"], D), "final.norm": mat(D, s=0.3)}
    for i, l in enumerate(cfg["layers"]):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        sd[p + "norm1"] = mat(D, s=0.3)
        sd[p + "canon1"] = mat(D, taps, s=0.4)
        if l["type"] == "latent_attention":
            H, d, dr, dv, r, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            sd.update({x + "dq": mat(qr, D), x + "dq.norm": near_one(qr), x + "uq": mat(H * (d + dr), qr),
                       x + "uk": mat(H * d, r), x + "uv": mat(H * dv, r), x + "o": mat(D, H * dv)})
            if m.get("kv_from") is None:
                sd.update({x + "dkv": mat(r + dr, D), x + "dkv.norm": near_one(r)})
        else:
            a, rr = m["left"], m["right"]
            H, G, d = a["heads"], a["kv_heads"], a["dim"]
            hd, lr = rr["heads"] * rr["dim"], ranks[i]
            sd.update({x + "left.q": mat(H * d, D), x + "left.q.b": mat(H * d), x + "left.k": mat(G * d, D),
                       x + "left.k.b": mat(G * d), x + "left.q.norm": near_one(d), x + "left.k.norm": near_one(d),
                       x + "left.pb": mat(H, s=1.0) - 1.0, x + "left.o": mat(D, H * d)})
            sd.update({x + "right." + n: mat(hd, D) for n in ("r", "k", "v", "g", "a")})
            sd.update({x + "right.a.b": mat(hd, s=1.0), x + "right.w1": mat(lr, D), x + "right.w2": mat(hd, lr, s=1.0),
                       x + "right.w0": mat(hd, s=1.0), x + "right.norm": near_one(hd), x + "right.o": mat(D, hd)})
        if l["mlp"] is not None:
            ff, y = l["mlp"]["ff"], p + "mlp."
            sd.update({p + "norm2": mat(D, s=0.3), p + "canon2": mat(D, taps, s=0.4), y + "gate": mat(ff, D),
                       y + "up": mat(ff, D), y + "down": mat(D, ff)})
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
