"""A plain, slow Kagolix forward pass in float64, one function per mechanism, written from the
design's equations.  It shares no code with the framework: the tests compare the framework's
kernels, caches and scheduler against it.

Notation: a sequence is a [T, D] matrix of rows x_t, t = 0 .. T-1 its positions; every function
takes the whole sequence and returns the whole output, recomputing everything from t = 0.
"""
import math

import torch

F = torch.float64


def group_rms(x, w, groups, eps):
    """Rows split into ``groups`` equal consecutive parts, each divided by sqrt(mean(part^2) + eps); times w."""
    T, D = x.shape
    p = x.reshape(T, groups, D // groups)
    p = p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)
    return p.reshape(T, D) * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def silu(z):
    return z * torch.sigmoid(z)


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    ap, an = softplus(p), 0.5 + softplus(q)
    return torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.expm1(torch.clamp(z, max=0)) - z) + 0.5 * z)


def causal_conv(x, w, b):
    """Per channel: out_t[c] = b[c] + sum_j w[c, taps-1-j] x_(t-j)[c], zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F) + b
    for t in range(T):
        for j in range(taps):
            if t - j >= 0:
                out[t] += w[:, taps - 1 - j] * x[t - j]
    return out


def attention(h, m, W, eps):
    """Chunk-local softmax attention with tanh-capped scores and a logarithmic distance penalty."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ W["q"].T
    k = h @ W["k"].T
    v = h @ W["v"].T
    q = group_rms(q, W["q.norm"], 1, eps).reshape(T, H, d)
    k = group_rms(k, W["k.norm"], 1, eps).reshape(T, G, d)
    v = v.reshape(T, G, dv)
    cap, size = m["softcap"], m["mask"]["size"]
    out = torch.zeros(T, H, dv, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            lo = (i // size) * size
            js = torch.arange(lo, i + 1)
            s = (k[lo:i + 1, g] @ q[i, hd]) * m["scale"]
            s = cap * torch.tanh(s / cap)
            s = s - W["r1"][hd] * torch.log1p(W["r2"][hd] * (i - js).to(F))
            p = torch.softmax(s, 0)
            out[i, hd] = p @ v[lo:i + 1, g]
    return out.reshape(T, H * dv) @ W["o"].T


def rglru(h, m, W):
    """Two branches; the recurrent one: conv, block-diagonal gates, S_t = a S_(t-1) + sqrt(1 - a^2) i u."""
    T = h.shape[0]
    y = gelu_tanh(h @ W["y"].T + W["y.b"])
    u = causal_conv(h @ W["x"].T + W["x.b"], W["conv"], W["conv.b"])
    nb = m["blocks"]
    bw = m["width"] // nb
    ub = u.reshape(T, nb, bw)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, W["ra"]) + W["ra.b"]).reshape(T, -1)
    ig = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, W["ri"]) + W["ri.b"]).reshape(T, -1)
    a = torch.exp(-8.0 * r * softplus(W["lam"]))
    S = torch.zeros(m["width"], dtype=F)
    out = torch.zeros(T, m["width"], dtype=F)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1 - a[t] ** 2) * ig[t] * u[t]
        out[t] = S
    return (out * y) @ W["o"].T


def mamba2(h, m, W, eps):
    """Selective state space per head: S_t = exp(-exp(A) dt) S_(t-1) + dt B x^T; y = S^T C + D x."""
    T = h.shape[0]
    nh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = nh * P
    zx = h @ W["in"].T
    z, xbc, dt = zx[:, :inner], zx[:, inner:2 * inner + 2 * G * N], zx[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W["conv"], W["conv.b"]))
    x = xbc[:, :inner].reshape(T, nh, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + W["dt_bias"])
    y = torch.zeros(T, nh, P, dtype=F)
    for hd in range(nh):
        g = hd // (nh // G)
        S = torch.zeros(N, P, dtype=F)
        for t in range(T):
            S = torch.exp(-torch.exp(W["A_log"][hd]) * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + W["D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = group_rms(y, W["norm"], m["norm_groups"], eps)
    return y @ W["o"].T


def dense_ff(h, W):
    return xielu(h @ W["up"].T, W["act"][0], W["act"][1]) @ W["down"].T


def moe_ff(h, mlp, W):
    """softmax router; the ``top`` largest of (score + correction) are chosen, weighted by the bare score."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.softmax(h @ W["router"].T, -1)
    choice = s + W["correction"]
    out = torch.zeros(h.shape[0], W["e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e in torch.topk(choice[t], top).indices.tolist():
            a = silu(h[t] @ W[f"e{e}.gate"].T) * (h[t] @ W[f"e{e}.up"].T)
            out[t] += s[t, e] * (a @ W[f"e{e}.down"].T)
    return out


def sub(sd, prefix):
    """Tensors below ``prefix`` with the prefix taken off, as float64."""
    return {k[len(prefix):]: v.to(F) for k, v in sd.items() if k.startswith(prefix)}


def forward(cfg, sd, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence from its first token."""
    eps, ng = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = sd["embed"].to(F)[torch.as_tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        W = sub(sd, p + "mix.")
        h = group_rms(x, sd[p + "norm1"].to(F), ng, eps)
        if layer["type"] == "attention":
            y = attention(h, layer["mixer"], W, eps)
        elif layer["type"] == "rglru":
            y = rglru(h, layer["mixer"], W)
        elif layer["type"] == "mamba2":
            y = mamba2(h, layer["mixer"], W, eps)
        else:
            raise ValueError(layer["type"])
        x = x + group_rms(y, sd[p + "norm1b"].to(F), ng, eps)
        if layer["mlp"] is not None:
            h = group_rms(x, sd[p + "norm2"].to(F), ng, eps)
            W = sub(sd, p + "mlp.")
            y = dense_ff(h, W) if layer["mlp"]["kind"] == "dense" else moe_ff(h, layer["mlp"], W)
            x = x + group_rms(y, sd[p + "norm2b"].to(F), ng, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    h = group_rms(x, sd["final.norm"].to(F), ng, eps)
    z = h @ sd["head"].to(F).T
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(z / cap)
