"""Sisavik layer execution on packed weight images and packed step batches.

Every layer of a Sisavik stack is

    x <- x + N1(mixer(C1(x)));   x <- x + N2(ff(C2(x)))          (the second line only with an ff)

with x the fp32 residual stream, C(h) = h + conv(h) a short causal convolution per channel over the
sequence (its last taps - 1 inputs are carried per request, for both sublayers of every layer) and
N(y) = y / sqrt(mean(y^2) + eps) * (1 + w) a norm on the sublayer's output only.  The mixer is

* ``latent_attention`` -- softmax attention over a sliding window whose keys and values are linear
  maps of one cached latent row c_j (RMS-normed) plus a rotated key part shared by all heads:
  score_h(i, j) = scale * (qn_h(i) . W_uk,h c_j + qr_h(i) . kr_j).  Only (c_j, kr_j) is cached.  Steps
  that continue a sequence fold the maps around the attention: the query side becomes
  qa_h = W_uk,h^T qn_h, the attention runs with one key/value head over the latent rows (keys [c | kr],
  values c), and W_uv,h maps the weighted latent of each head to its value size.  Whole prompts make
  per-head keys and values from the step's cached rows instead (fewer products per key, and head
  sizes the matrix-core attention serves).  A layer with ``kv_from`` reads another layer's latent rows
  instead of writing its own;
* ``parallel`` -- two mixers on the same input, summed with weights from the config: a grouped-query
  attention whose values are the keys as projected (before their norm and rotation), whose weights
  are sigmoid(score + b_h) without normalisation over the keys, and which sees a sliding window plus
  the first ``keep_first`` tokens; beside it a generalized delta rule, per head a state S [key, value]:
  S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t, with u the unit
  key, w a learned decay and a a removal rate; o is RMS-normed per head, weighted and gated.

The feed-forward is W_down(gelu_tanh(W_gate h) * W_up h).  Each mechanism is an op of the backend
(``ops/hip_seq.py``: the kernels of ``csrc/kernels/seq``; ``ops/torch_seq.py`` on the CPU) with its
constants as arguments; this file only strings them together.  Latent rows, keys and recurrent
states live in :class:`~..runtime.seq_state.SequenceStateCache`.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch

from .kagolix import HybridContext  # noqa: F401  (the context the engine builds for every hybrid family)
from .layout import LayerLayout, Placement, layer_kind, spec_layout, spec_placements

F32 = "f32"
DECAY_SCALE = math.exp(-0.5)       # w = exp(-DECAY_SCALE * sigmoid(.)): a decay between exp(-0.607) and 1
UNIT_KEY_EPS = 1e-6                # u = k / sqrt(sum(k^2) + UNIT_KEY_EPS)


def _latent_cols(m: dict):
    return int(m["q_rank"]), int(m["kv_rank"]), int(m["rot_dim"])


def _parallel_cols(m: dict) -> Dict[str, tuple]:
    """Column ranges (start, width) of the stacked input projection of a parallel mixer."""
    a, r = m["left"], m["right"]
    hd = r["heads"] * r["dim"]
    widths = [("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"]), ("r", hd), ("rk", hd), ("rv", hd),
              ("g", hd), ("a", hd), ("w1", int(r["decay_rank"]))]
    out, at = {}, 0
    for n, w in widths:
        out[n] = (at, w)
        at += w
    out["all"] = (0, at)
    return out


def _specs(cfg, name: str):
    """[(slot, shape, dtype tag, [(checkpoint tensor, element offset in the slot, shape[, options])])]."""
    D, V = cfg.width, cfg.vocab
    kind = layer_kind(name)
    if kind == "embed":
        return [("embed", (V, D), None, [("embed", 0, (V, D))])]
    if kind == "head":
        return [("head", (V, D), None, [("head", 0, (V, D))])]
    if kind == "norm":
        return [("norm", (D,), F32, [("final.norm", 0, (D,))])]
    L, p, taps = cfg.layer(name), name + ".", cfg.canon_taps
    m, x = L.mixer, name + ".mix."
    out = [("norm1", (D,), F32, [(p + "norm1", 0, (D,))]), ("canon1", (D, taps), F32, [(p + "canon1", 0, (D, taps))])]
    if L.type == "latent_attention":
        qr, r, dr = _latent_cols(m)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        parts = [(x + "dq", 0, (qr, D))]
        if m.get("kv_from") is None:
            parts.append((x + "dkv", qr * D, (r + dr, D)))
            out.append(("dkvn", (r,), F32, [(x + "dkv.norm", 0, (r,))]))
        out += [("wdqkv", (sum(s[2][0] for s in parts), D), None, parts),
                ("dqn", (qr,), F32, [(x + "dq.norm", 0, (qr,))]),
                ("wuq", (H * (d + dr), qr), None, [(x + "uq", 0, (H * (d + dr), qr))]),
                # W_uk per head, transposed: the product that folds it into the queries reads it as [N = r, K = d]
                ("wukt", (H, r, d), None, [(x + "uk", 0, (H * d, r), {"view": (H, d, r), "perm": (0, 2, 1)})]),
                ("wuk", (H, d, r), None, [(x + "uk", 0, (H * d, r))]),
                ("wuv", (H, dv, r), None, [(x + "uv", 0, (H * dv, r))]),
                ("wo", (D, H * dv), None, [(x + "o", 0, (D, H * dv))])]
    elif L.type == "parallel":
        a, r = m["left"], m["right"]
        c = _parallel_cols(m)
        n_in = c["all"][1]
        H, d, hd = a["heads"], a["dim"], r["heads"] * r["dim"]
        lo, ro = H * a["vdim"], hd
        out += [("win", (n_in, D), None,
                 [(x + "left.q", c["q"][0] * D, (c["q"][1], D)), (x + "left.k", c["k"][0] * D, (c["k"][1], D)),
                  (x + "right.r", c["r"][0] * D, (hd, D)), (x + "right.k", c["rk"][0] * D, (hd, D)),
                  (x + "right.v", c["rv"][0] * D, (hd, D)), (x + "right.g", c["g"][0] * D, (hd, D)),
                  (x + "right.a", c["a"][0] * D, (hd, D)), (x + "right.w1", c["w1"][0] * D, (c["w1"][1], D))]),
                ("bin", (n_in,), F32, [(x + "left.q.b", c["q"][0], (c["q"][1],)), (x + "left.k.b", c["k"][0], (c["k"][1],)),
                                        (x + "right.a.b", c["a"][0], (hd,))]),
                ("lqn", (d,), F32, [(x + "left.q.norm", 0, (d,))]), ("lkn", (d,), F32, [(x + "left.k.norm", 0, (d,))]),
                ("lpb", (H,), F32, [(x + "left.pb", 0, (H,))]),
                ("rw2", (hd, c["w1"][1]), None, [(x + "right.w2", 0, (hd, c["w1"][1]))]),
                ("rw0", (hd,), F32, [(x + "right.w0", 0, (hd,))]), ("rnorm", (hd,), F32, [(x + "right.norm", 0, (hd,))]),
                # [left.o | right.o] side by side: one product over the two mixers' concatenated outputs
                ("wo", (D, lo + ro), None, [(x + "left.o", 0, (D, lo), {"ld": lo + ro}),
                                            (x + "right.o", lo, (D, ro), {"ld": lo + ro})])]
    else:
        raise NotImplementedError(L.type)
    if L.mlp is not None:
        ff, y = L.mlp["ff"], p + "mlp."
        out += [("norm2", (D,), F32, [(p + "norm2", 0, (D,))]), ("canon2", (D, taps), F32, [(p + "canon2", 0, (D, taps))]),
                ("wgu", (2 * ff, D), None, [(y + "gate", 0, (ff, D)), (y + "up", ff * D, (ff, D))]),
                ("wdown", (D, ff), None, [(y + "down", 0, (D, ff))])]
    return out


def layout(cfg, name: str, elem_size: int = 2) -> LayerLayout:
    return spec_layout(layer_kind(name), _specs(cfg, name), elem_size)


def placements(cfg, name: str, elem_size: int = 2) -> List[Placement]:
    return spec_placements(layout(cfg, name, elem_size), _specs(cfg, name), elem_size)


def state_spec(cfg) -> dict:
    """What a request keeps between steps: per latent attention layer with a latent of its own one
    pool of rows [c | kr]; per parallel layer the left mixer's keys and values and the right mixer's
    state; per layer the last taps - 1 inputs of its two input convolutions."""
    paged, alias, slots, horizons = {}, {}, {}, []
    D, taps = cfg.width, cfg.canon_taps
    for i, l in enumerate(cfg.layers):
        name, m = f"l{i}", l.mixer
        slots[name] = {"canon1": (taps - 1, D)}
        if l.mlp is not None:
            slots[name]["canon2"] = (taps - 1, D)
        if l.type == "latent_attention":
            if cfg.kv_owner(i) == i:
                paged[name] = {"ckr": int(m["kv_rank"]) + int(m["rot_dim"])}
            else:
                alias[name] = f"l{cfg.kv_owner(i)}"
            horizons.append(("window", int(m["mask"]["size"]), 0))
        else:
            a, r = m["left"], m["right"]
            paged[name] = {"k": a["kv_heads"] * a["dim"], "v": a["kv_heads"] * a["dim"]}
            horizons.append(("window", int(a["mask"]["size"]), int(a["mask"].get("keep_first", 0))))
            slots[name]["state"] = (r["heads"], r["dim"], r["dim"])
    return {"paged": paged, "alias": alias, "slots": slots, "horizons": horizons}


# ------------------------------------------------------------------------------------ execution
def _latent_attention(ctx, m: dict, W, h, meta, name: str):
    ops, eps, cdt = ctx.ops, ctx.cfg.norm_eps, ctx.compute_dtype
    qr, r, dr = _latent_cols(m)
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    rot = (int(m["rot"]["dims"]), float(m["rot"]["base"]))
    pool = ctx.cache.pools(name)["ckr"]                                  # [pages, page, c | kr]
    z = ops.matmul_nt(h, W["wdqkv"])                                      # fp32 [T, c_q (| c_kv | k_rot)]
    if m.get("kv_from") is None:
        rows = pool.view(-1, r + dr)
        ops.head_norm_rope(z, 1, r, qr, 0, rows, 0, 0, meta, w=W["dkvn"], eps=eps, row_map=meta["kv_slot"])
        ops.head_norm_rope(z, 1, dr, qr + r, 0, rows, r, 0, meta, rot=rot, row_map=meta["kv_slot"])
    cq = ops.group_rmsnorm(z[:, :qr], W["dqn"], 1, eps, out_dtype=cdt)
    q = ops.matmul_nt(cq, W["wuq"])                                       # fp32 [T, H (d | dr)]
    T, window = q.shape[0], int(m["mask"]["size"])
    local = meta.get("local_table")
    if local is not None and ops.unfolded_attention_ok(d + dr, dv, cdt):
        # whole prompts (every request of the step starts at position 0, so all keys are this step's
        # rows): keys and values are made per head from the rows as cached, [W_uk,h c | kr] and W_uv,h c,
        # and the attention runs over them in the step's own row order (pages of one row)
        ckr = ops.gather_rows(pool.view(-1, r + dr), meta["kv_slot"])     # [T, c | kr]
        kf = torch.empty(T, H * (d + dr), dtype=cdt, device=q.device)
        ops.head_matmul_nt(ckr, W["wuk"], H, 0, kf, d + dr)
        ops.head_norm_rope(ckr, H, dr, r, 0, kf, d, d + dr, meta)         # the one rotated part beside every head's keys
        vf = ops.matmul_nt(ckr[:, :r], W["wuv"].view(H * dv, r), out_dtype=cdt)
        ops.head_norm_rope(q, H, dr, d, d + dr, q, d, d + dr, meta, rot=rot)          # (in place)
        o = ops.attn_paged(q, kf.view(T, 1, -1), vf.view(T, 1, -1), dict(meta, page_table=local), H, H, d + dr, dv,
                           scale=float(m["scale"]), softcap=0.0, r1=None, r2=None, chunk=0, page_size=1, out_dtype=cdt,
                           window=window)
        return ops.matmul_nt(o, W["wo"])
    # otherwise (decoding, portions): the maps are folded around the attention.  The query each head asks
    # the latent rows with: [W_uk,h^T q_unrotated | q_rotated]
    qa = torch.empty(T, H * (r + dr), dtype=torch.float32, device=q.device)
    ops.head_matmul_nt(q, W["wukt"], H, d + dr, qa, r + dr)
    ops.head_norm_rope(q, H, dr, d, d + dr, qa, r, r + dr, meta, rot=rot)
    a = ops.attn_paged(qa, pool, pool, meta, H, 1, r + dr, r, scale=float(m["scale"]), softcap=0.0, r1=None, r2=None,
                       chunk=0, page_size=ctx.cache.page_size, out_dtype=cdt, window=window)
    o = torch.empty(T, H * dv, dtype=cdt, device=q.device)
    ops.head_matmul_nt(a, W["wuv"], H, r, o, dv)                          # each head's weighted latent -> its values
    return ops.matmul_nt(o, W["wo"])


def _parallel(ctx, m: dict, W, h, meta, name: str):
    ops, eps, cdt = ctx.ops, ctx.cfg.norm_eps, ctx.compute_dtype
    a, r = m["left"], m["right"]
    H, G, d = a["heads"], a["kv_heads"], a["dim"]
    Hr, dr = r["heads"], r["dim"]
    c = _parallel_cols(m)
    col = lambda z, n: z[:, c[n][0]:c[n][0] + c[n][1]]
    rot = (int(a["rot"]["dims"]), float(a["rot"]["base"]))
    T = h.shape[0]
    z = ops.matmul_nt(h, W["win"], bias=W["bin"])                         # fp32 [T, q | k | r | k | v | g | a | w1]
    both = torch.empty(T, H * d + Hr * dr, dtype=cdt, device=h.device)    # [left | right] mixer outputs, weighted
    # left: q and k normed per head and rotated; the keys as projected are the values
    pools = ctx.cache.pools(name)
    kc, vc = pools["k"], pools["v"]
    q = torch.empty(T, H * d, dtype=torch.float32, device=h.device)
    ops.head_norm_rope(z, H, d, c["q"][0], d, q, 0, d, meta, w=W["lqn"], eps=eps, rot=rot)
    ops.head_norm_rope(z, G, d, c["k"][0], d, kc.view(-1, G * d), 0, d, meta, w=W["lkn"], eps=eps, rot=rot,
                       row_map=meta["kv_slot"], raw=vc.view(-1, G * d))
    ops.attn_paged(q, kc, vc, meta, H, G, d, d, scale=float(a["scale"]), softcap=0.0, r1=None, r2=None, chunk=0,
                   page_size=ctx.cache.page_size, out_dtype=cdt, window=int(a["mask"]["size"]),
                   keep_first=int(a["mask"].get("keep_first", 0)), gate_bias=W["lpb"], out_scale=float(m["left_scale"]),
                   out=both[:, :H * d])
    # right: the decay's small two-layer map, then the recurrence with its gates, norm and output gate fused
    wz = ops.matmul_nt(ops.unary(col(z, "w1"), "tanh", cdt), W["rw2"])    # fp32 [T, Hr dr], before + w0
    st = ctx.cache.recurrent(name)["state"]
    ops.delta_rule_scan(col(z, "r"), col(z, "rk"), col(z, "rv"), col(z, "a"), wz, col(z, "g"), W["rw0"], W["rnorm"], st,
                        meta, Hr, dr, decay_scale=DECAY_SCALE, key_eps=UNIT_KEY_EPS, norm_eps=eps,
                        out_scale=float(m["right_scale"]), out=both[:, H * d:])
    return ops.matmul_nt(both, W["wo"])


def run_block(ctx, W, x: torch.Tensor, meta: dict, name: str) -> torch.Tensor:
    cfg, ops, cdt = ctx.cfg, ctx.ops, ctx.compute_dtype
    L = cfg.layer(name)
    eps = cfg.norm_eps
    st = ctx.cache.recurrent(name)
    h = ops.causal_conv(x, W["canon1"], None, st["canon1"], meta, residual=True, out_dtype=cdt)
    y = {"latent_attention": _latent_attention, "parallel": _parallel}[L.type](ctx, L.mixer, W, h, meta, name)
    ops.add_group_rmsnorm_(x, y, W["norm1"], 1, eps, w_offset=1.0)
    if L.mlp is not None:
        h = ops.causal_conv(x, W["canon2"], None, st["canon2"], meta, residual=True, out_dtype=cdt)
        gu = ops.matmul_nt(h, W["wgu"])                                   # fp32 [T, gate | up]
        y = ops.matmul_nt(ops.gate_mul(gu, cdt, act="gelu_tanh"), W["wdown"])
        ops.add_group_rmsnorm_(x, y, W["norm2"], 1, eps, w_offset=1.0)
    return x


def run_layer(ctx, name: str, W: Dict[str, torch.Tensor], state, batch, meta: dict) -> torch.Tensor:
    """One layer of the stack on a step batch: the residual rows in, the residual rows out (fp32);
    ``final.norm`` keeps the rows whose logits are wanted, ``head`` returns their logits."""
    cfg, ops = ctx.cfg, ctx.ops
    kind = layer_kind(name)
    if kind == "embed":
        out, ctx.embed_out = ctx.embed_out, None
        return ops.embed_rows(meta["ids"], W["embed"], out=out)
    if kind == "decoder":
        return run_block(ctx, W, state, meta, name)
    if kind == "norm":
        return ops.group_rmsnorm(state, W["norm"], 1, cfg.norm_eps, out_dtype=ctx.compute_dtype,
                                 row_idx=meta["want_idx"], w_offset=1.0)
    return ops.matmul_nt(state, W["head"])


def layer_flops(cfg, name: str, rows: int, ctx_keys: float = 0.0) -> float:
    """Approximate forward FLOPs of decoder layer ``name`` on ``rows`` tokens (matrix products; the
    attention's score and value products over ``ctx_keys`` visible keys per row on average)."""
    L, D = cfg.layer(name), cfg.width
    m = L.mixer
    if L.type == "latent_attention":
        qr, r, dr = _latent_cols(m)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        own = (r + dr) if m.get("kv_from") is None else 0
        f = 2.0 * rows * (D * (qr + own) + qr * H * (d + dr) + H * d * r + H * r * dv + H * dv * D)
        f += 2.0 * rows * min(ctx_keys, float(m["mask"]["size"])) * H * (2 * r + dr)
    else:
        a, r = m["left"], m["right"]
        c = _parallel_cols(m)
        hd = r["heads"] * r["dim"]
        f = 2.0 * rows * (D * c["all"][1] + c["w1"][1] * hd + (a["heads"] * a["dim"] + hd) * D)
        f += 4.0 * rows * min(ctx_keys, float(a["mask"]["size"] + a["mask"].get("keep_first", 0))) * a["heads"] * a["dim"]
        f += 8.0 * rows * hd * r["dim"]
    if L.mlp is not None:
        f += 6.0 * rows * D * L.mlp["ff"]
    return f
