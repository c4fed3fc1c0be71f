"""Kagolix layer execution on packed weight images and packed step batches.

A Kagolix model is a stack of unlike layers.  Every layer is

    x <- x + N1b(mixer(N1(x)));   x <- x + N2b(ff(N2(x)))        (the second line only with an ff)

with N* a group RMS norm (the row cut into ``norm.groups`` equal parts, each scaled by its own
1 / sqrt(mean(part^2) + eps), times a weight) and the residual stream x in fp32.  The mixer is one of

* ``attention``  — grouped-query softmax attention without rotation: q and k are RMS-normed over
  their whole projection; score = cap * tanh(scale * q.k / cap) - r1_h * ln(1 + r2_h * (i - j));
  query i sees key j <= i of its own chunk of ``mask.size`` positions (chunks count from position 0);
* ``rglru``      — a gated branch gelu(W_y h + b) times a linear recurrence over conv(W_x h + b):
  S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-8 r_t softplus(lam)) and r, i
  block-diagonal sigmoid gates of u;
* ``mamba2``     — a selective state-space layer, S_t = exp(-exp(A) dt_t) S_(t-1) + dt_t B_t x_t^T,
  y_t = S_t^T C_t + D x_t, gated by silu(z) and group-normed before the output projection;

and the feed-forward is dense (W_down xIELU(W_up h)) or a mixture of SiLU-gated experts chosen by
softmax score plus a per-expert correction and weighted by the bare score.

Each mechanism is an op of the backend (``ops/hip_seq.py``: the kernels of ``csrc/kernels/seq``;
``ops/torch_seq.py`` on the CPU) with its constants as arguments; this file only strings them
together.  K/V pages and recurrent states live in :class:`~..runtime.seq_state.SequenceStateCache`,
a step's rows and their places in it come packed in a :class:`~..runtime.batch.StepBatch`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .layout import LayerLayout, Placement, layer_kind, spec_layout, spec_placements

F32 = "f32"


def _attn_cols(m: dict):
    return m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]


def _mamba_cols(m: dict):
    inner = m["heads"] * m["vdim"]
    gn = m["groups"] * m["state"]
    return inner, gn, 2 * inner + 2 * gn + m["heads"]


def _specs(cfg, name: str):
    """[(slot, shape, dtype tag, [(checkpoint tensor, element offset in the slot, shape)])]."""
    D, V = cfg.width, cfg.vocab
    kind = layer_kind(name)
    if kind == "embed":
        return [("embed", (V, D), None, [("embed", 0, (V, D))])]
    if kind == "head":
        return [("head", (V, D), None, [("head", 0, (V, D))])]
    if kind == "norm":
        return [("norm", (D,), F32, [("final.norm", 0, (D,))])]
    L, p = cfg.layer(name), name + "."
    m = L.mixer
    out = [(n, (D,), F32, [(p + n, 0, (D,))]) for n in ("norm1", "norm1b")]
    x = p + "mix."
    if L.type == "attention":
        qs, ks, vs = _attn_cols(m)
        H = m["heads"]
        out += [("wqkv", (qs + ks + vs, D), None, [(x + "q", 0, (qs, D)), (x + "k", qs * D, (ks, D)),
                                                     (x + "v", (qs + ks) * D, (vs, D))]),
                ("qn", (qs,), F32, [(x + "q.norm", 0, (qs,))]), ("kn", (ks,), F32, [(x + "k.norm", 0, (ks,))]),
                ("r1", (H,), F32, [(x + "r1", 0, (H,))]), ("r2", (H,), F32, [(x + "r2", 0, (H,))]),
                ("wo", (D, H * m["vdim"]), None, [(x + "o", 0, (D, H * m["vdim"]))])]
    elif L.type == "rglru":
        Wd, nb, taps = m["width"], m["blocks"], m["conv"]
        bw = Wd // nb
        out += [("wyx", (2 * Wd, D), None, [(x + "y", 0, (Wd, D)), (x + "x", Wd * D, (Wd, D))]),
                ("byx", (2 * Wd,), F32, [(x + "y.b", 0, (Wd,)), (x + "x.b", Wd, (Wd,))]),
                ("conv", (Wd, taps), F32, [(x + "conv", 0, (Wd, taps))]),
                ("convb", (Wd,), F32, [(x + "conv.b", 0, (Wd,))]),
                ("wg", (2 * nb, bw, bw), None, [(x + "ra", 0, (nb, bw, bw)), (x + "ri", nb * bw * bw, (nb, bw, bw))]),
                ("bg", (2 * Wd,), F32, [(x + "ra.b", 0, (nb, bw)), (x + "ri.b", Wd, (nb, bw))]),
                ("lam", (Wd,), F32, [(x + "lam", 0, (Wd,))]),
                ("wo", (D, Wd), None, [(x + "o", 0, (D, Wd))])]
    elif L.type == "mamba2":
        inner, gn, n_in = _mamba_cols(m)
        C, nh, taps = inner + 2 * gn, m["heads"], m["conv"]
        out += [("win", (n_in, D), None, [(x + "in", 0, (n_in, D))]),
                ("conv", (C, taps), F32, [(x + "conv", 0, (C, taps))]),
                ("convb", (C,), F32, [(x + "conv.b", 0, (C,))]),
                ("dt_bias", (nh,), F32, [(x + "dt_bias", 0, (nh,))]),
                ("A_log", (nh,), F32, [(x + "A_log", 0, (nh,))]), ("Dskip", (nh,), F32, [(x + "D", 0, (nh,))]),
                ("mnorm", (inner,), F32, [(x + "norm", 0, (inner,))]),
                ("wo", (D, inner), None, [(x + "o", 0, (D, inner))])]
    else:
        raise NotImplementedError(L.type)
    if L.mlp is not None:
        out += [(n, (D,), F32, [(p + n, 0, (D,))]) for n in ("norm2", "norm2b")]
        y = p + "mlp."
        if L.mlp["kind"] == "dense":
            ff = L.mlp["ff"]
            out += [("wup", (ff, D), None, [(y + "up", 0, (ff, D))]), ("wdown", (D, ff), None, [(y + "down", 0, (D, ff))]),
                    ("act", (2,), F32, [(y + "act", 0, (2,))])]
        else:
            E, ff = L.mlp["router"]["experts"], L.mlp["expert"]["ff"]
            gu, dn = [], []
            for e in range(E):
                gu += [(f"{y}e{e}.gate", e * 2 * ff * D, (ff, D)), (f"{y}e{e}.up", (e * 2 + 1) * ff * D, (ff, D))]
                dn.append((f"{y}e{e}.down", e * D * ff, (D, ff)))
            out += [("wrouter", (E, D), None, [(y + "router", 0, (E, D))]),
                    ("corr", (E,), F32, [(y + "correction", 0, (E,))]),
                    ("wgu", (E, 2 * ff, D), None, gu), ("wdown", (E, D, ff), None, dn)]
    return out


def kagolix_layout(cfg, name: str, elem_size: int = 2) -> LayerLayout:
    return spec_layout(layer_kind(name), _specs(cfg, name), elem_size)


def kagolix_placements(cfg, name: str, elem_size: int = 2) -> List[Placement]:
    """Where every checkpoint tensor of layer ``name`` lands in its image (stacked projections are
    whole tensors back to back: [q; k; v], [y; x], [ra; ri], per expert [gate; up])."""
    return spec_placements(kagolix_layout(cfg, name, elem_size), _specs(cfg, name), elem_size)


layout, placements = kagolix_layout, kagolix_placements      # (the names models.hybrid_family expects)


def state_spec(cfg) -> dict:
    """What a request keeps between steps (runtime.seq_state.SequenceStateCache): per attention layer
    paged keys and values and how far back it looks, per recurrent layer fp32 slot tensors."""
    paged, slots, horizons = {}, {}, []
    for i, l in enumerate(cfg.layers):
        name, m = f"l{i}", l.mixer
        if l.type == "attention":
            paged[name] = {"k": m["kv_heads"] * m["dim"], "v": m["kv_heads"] * m["vdim"]}
            horizons.append(("chunk", int(m["mask"]["size"]), 0))
        elif l.type == "rglru":
            slots[name] = {"conv": (m["conv"] - 1, m["width"]), "state": (m["width"],)}
        elif l.type == "mamba2":
            inner = m["heads"] * m["vdim"]
            slots[name] = {"conv": (m["conv"] - 1, inner + 2 * m["groups"] * m["state"]),
                           "state": (m["heads"], m["state"], m["vdim"])}
    return {"paged": paged, "slots": slots, "horizons": horizons}


# ------------------------------------------------------------------------------------ execution
@dataclass
class HybridContext:
    """What a hybrid layer needs besides its weights: the op backend, the GEMM element type
    (bf16, or fp32 for the all-32-bit mode) and the per-request state."""
    cfg: object
    ops: object
    device: torch.device
    compute_dtype: torch.dtype
    cache: Optional[object] = None           # runtime.seq_state.SequenceStateCache
    embed_out: Optional[torch.Tensor] = None
    act_dtype: torch.dtype = torch.float32   # the residual stream
    # (fields the engine's pass machinery reads on every context)
    prune_last: bool = False
    last_decoder: str = ""
    ws: Optional[object] = None
    row_exact: bool = False
    fused_norm: bool = False
    prefix_entry: Optional[object] = None
    mlp_chunk: int = 0
    attn_rows: int = 0
    qkv_chunk: int = 0


def _attention(ctx, m: dict, W, h, meta, name: str):
    ops, eps, cdt = ctx.ops, ctx.cfg.norm_eps, ctx.compute_dtype
    qs, ks, vs = _attn_cols(m)
    qkv = ops.matmul_nt(h, W["wqkv"])                                     # fp32 [T, q | k | v]
    q = ops.group_rmsnorm(qkv[:, :qs], W["qn"], 1, eps, out_dtype=cdt)    # over the whole projection
    kc, vc = ctx.cache.kv(name)
    ops.kv_store(qkv[:, qs:qs + ks], W["kn"], eps, qkv[:, qs + ks:], kc, vc, meta["kv_slot"])
    a = ops.attn_paged(q, kc, vc, meta, m["heads"], m["kv_heads"], m["dim"], m["vdim"], scale=float(m["scale"]),
                       softcap=float(m["softcap"]), r1=W["r1"], r2=W["r2"], chunk=int(m["mask"]["size"]),
                       page_size=ctx.cache.page_size, out_dtype=cdt)
    return ops.matmul_nt(a, W["wo"])


def _rglru(ctx, m: dict, W, h, meta, name: str):
    ops, cdt = ctx.ops, ctx.compute_dtype
    Wd = m["width"]
    st = ctx.cache.recurrent(name)
    yx = ops.matmul_nt(h, W["wyx"], bias=W["byx"])                        # fp32 [T, y | x]
    u = ops.causal_conv(yx[:, Wd:], W["conv"], W["convb"], st["conv"], meta, act="none")
    g = ops.block_linear(u, W["wg"], W["bg"], m["blocks"], cdt)           # fp32 [T, r | i] before the sigmoid
    a = ops.rglru_scan(u, g, W["lam"], yx[:, :Wd], st["state"], meta, c=8.0, out_dtype=cdt)
    return ops.matmul_nt(a, W["wo"])


def _mamba2(ctx, m: dict, W, h, meta, name: str):
    ops, cdt = ctx.ops, ctx.compute_dtype
    inner, gn, n_in = _mamba_cols(m)
    st = ctx.cache.recurrent(name)
    zx = ops.matmul_nt(h, W["win"])                                       # fp32 [T, z | x | B | C | dt]
    xbc = ops.causal_conv(zx[:, inner:2 * inner + 2 * gn], W["conv"], W["convb"], st["conv"], meta, act="silu")
    y = ops.ssd_scan(xbc, zx[:, :inner], zx[:, 2 * inner + 2 * gn:], W["dt_bias"], W["A_log"], W["Dskip"],
                     st["state"], meta, m["heads"], m["vdim"], m["state"], m["groups"])   # fp32, gated by silu(z)
    a = ops.group_rmsnorm(y, W["mnorm"], m["norm_groups"], ctx.cfg.norm_eps, out_dtype=cdt)
    return ops.matmul_nt(a, W["wo"])


def _moe(ctx, mlp: dict, W, h):
    ops, cdt = ctx.ops, ctx.compute_dtype
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = ops.matmul_nt(h, W["wrouter"])                               # fp32 accumulation of the rows
    route = ops.moe_route_corrected(logits, W["corr"], top)
    hp = ops.gather_rows(h, route.rows)                                   # rows sorted by expert
    gu = ops.grouped_matmul_nt(hp, W["wgu"], route.offs)                  # fp32 [T top, gate | up]
    a = ops.silu_mul(gu, out_dtype=cdt)
    yo = ops.grouped_matmul_nt(a, W["wdown"], route.offs)
    return ops.moe_weighted_sum(yo, route)                                # fp32 [T, D]


def run_block(ctx, W, x: torch.Tensor, meta: dict, name: str) -> torch.Tensor:
    cfg, ops, cdt = ctx.cfg, ctx.ops, ctx.compute_dtype
    L = cfg.layer(name)
    ng, eps = cfg.norm_groups, cfg.norm_eps
    h = ops.group_rmsnorm(x, W["norm1"], ng, eps, out_dtype=cdt)
    y = {"attention": _attention, "rglru": _rglru, "mamba2": _mamba2}[L.type](ctx, L.mixer, W, h, meta, name)
    ops.add_group_rmsnorm_(x, y, W["norm1b"], ng, eps)
    if L.mlp is not None:
        h = ops.group_rmsnorm(x, W["norm2"], ng, eps, out_dtype=cdt)
        if L.mlp["kind"] == "dense":
            # (the activation and the rounding for the down projection happen in the up projection's epilogue)
            y = ops.matmul_nt(ops.matmul_nt(h, W["wup"], xielu=W["act"], out_dtype=cdt), W["wdown"])
        else:
            y = _moe(ctx, L.mlp, W, h)
        ops.add_group_rmsnorm_(x, y, W["norm2b"], ng, eps)
    return x


def run_layer(ctx, name: str, W: Dict[str, torch.Tensor], state, batch, meta: dict) -> torch.Tensor:
    """One layer of the stack on a step batch: the residual rows in, the residual rows out (fp32);
    ``final.norm`` keeps the rows whose logits are wanted, ``head`` returns their capped logits."""
    cfg, ops = ctx.cfg, ctx.ops
    kind = layer_kind(name)
    if kind == "embed":
        out, ctx.embed_out = ctx.embed_out, None
        return ops.embed_rows(meta["ids"], W["embed"], out=out)
    if kind == "decoder":
        return run_block(ctx, W, state, meta, name)
    if kind == "norm":
        return ops.group_rmsnorm(state, W["norm"], cfg.norm_groups, cfg.norm_eps, out_dtype=ctx.compute_dtype,
                                 row_idx=meta["want_idx"])
    z = ops.matmul_nt(state, W["head"])
    return ops.softcap_(z, cfg.logit_softcap)


def layer_flops(cfg, name: str, rows: int, ctx_keys: float = 0.0) -> float:
    """Approximate forward FLOPs of decoder layer ``name`` on ``rows`` tokens (matrix products; the
    attention's score and value products over ``ctx_keys`` visible keys per row on average)."""
    L, D = cfg.layer(name), cfg.width
    m = L.mixer
    if L.type == "attention":
        qs, ks, vs = _attn_cols(m)
        f = 2.0 * rows * D * (qs + ks + vs + m["heads"] * m["vdim"]) + 2.0 * rows * ctx_keys * (qs + m["heads"] * m["vdim"])
    elif L.type == "rglru":
        f = 2.0 * rows * (3 * D * m["width"] + 2 * m["width"] * m["width"] // m["blocks"])
    else:
        inner, gn, n_in = _mamba_cols(m)
        f = 2.0 * rows * (D * (n_in + inner) + 3 * inner * m["state"])
    if L.mlp is not None:
        if L.mlp["kind"] == "dense":
            f += 4.0 * rows * D * L.mlp["ff"]
        else:
            f += 2.0 * rows * D * (L.mlp["router"]["experts"] + 3 * L.mlp["router"]["top"] * L.mlp["expert"]["ff"])
    return f
