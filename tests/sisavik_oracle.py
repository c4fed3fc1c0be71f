"""A plain, slow Sisavik forward pass in float64, one function per mechanism, written from the
design's equations.  It shares no code with the framework: the tests compare the framework's
kernels, caches and scheduler against it.

Notation: a sequence is a [T, D] matrix of rows x_t, t = 0 .. T-1 its positions; every function
takes the whole sequence and returns the whole output, recomputing everything from t = 0.
"""
import math

import torch

F = torch.float64


def rms(x, eps):
    """Rows divided by sqrt(mean(row^2) + eps)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def input_conv(h, w):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j), rows before the start are zeros."""
    T, C = h.shape
    taps = w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate(x, pos, dims, base):
    """x: [T, heads, d].  The first ``dims`` entries of each head turn in pairs (2i, 2i + 1) by the
    angle pos * base^(-2i / dims); the rest stay."""
    out = x.clone()
    for i in range(dims // 2):
        a = pos.to(F) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


def sees(i, j, size, keep_first=0):
    return j <= i and (i - j < size or j < keep_first)


def latent_kv(h, m, W, eps):
    """The cached part of a latent attention layer: the normed latent and the one rotated key part."""
    T = h.shape[0]
    r, dr = m["kv_rank"], m["rot_dim"]
    ckv = h @ W["dkv"].T
    c = rms(ckv[:, :r], eps) * W["dkv.norm"]
    pos = torch.arange(T)
    kr = rotate(ckv[:, r:].reshape(T, 1, dr), pos, m["rot"]["dims"], m["rot"]["base"]).reshape(T, dr)
    return c, kr


def latent_attention(h, m, W, eps, shared=None):
    """Softmax attention over a sliding window with keys and values made from a cached latent;
    ``shared`` = (c, kr) of the layer whose latent this layer reads."""
    T = h.shape[0]
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms(h @ W["dq"].T, eps) * W["dq.norm"]
    q = (cq @ W["uq"].T).reshape(T, H, d + dr)
    pos = torch.arange(T)
    qn = q[:, :, :d]
    qr = rotate(q[:, :, d:], pos, m["rot"]["dims"], m["rot"]["base"])
    c, kr = shared if shared is not None else latent_kv(h, m, W, eps)
    kn = (c @ W["uk"].T).reshape(T, H, d)
    v = (c @ W["uv"].T).reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F)
    size = m["mask"]["size"]
    for i in range(T):
        js = [j for j in range(T) if sees(i, j, size)]
        for hh in range(H):
            s = torch.stack([(qn[i, hh] @ kn[j, hh] + qr[i, hh] @ kr[j]) * m["scale"] for j in js])
            p = torch.softmax(s, 0)
            out[i, hh] = (p[:, None] * v[js, hh]).sum(0)
    return out.reshape(T, H * dv) @ W["o"].T


def sigmoid_attention(h, m, W, eps):
    """Grouped-query attention whose values are the keys as projected; q and k normed per head and
    rotated; every visible key weighs sigmoid(score + pb_h), without normalisation over the keys."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ W["q"].T + W["q.b"]).reshape(T, H, d)
    k = (h @ W["k"].T + W["k.b"]).reshape(T, G, d)
    v = k.clone()
    pos = torch.arange(T)
    q = rotate(rms(q, eps) * W["q.norm"], pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate(rms(k, eps) * W["k.norm"], pos, m["rot"]["dims"], m["rot"]["base"])
    size, keep = m["mask"]["size"], m["mask"].get("keep_first", 0)
    out = torch.zeros(T, H, d, dtype=F)
    for i in range(T):
        for j in range(T):
            if sees(i, j, size, keep):
                for hh in range(H):
                    g = hh // (H // G)
                    out[i, hh] += torch.sigmoid((q[i, hh] @ k[j, g]) * m["scale"] + W["pb"][hh]) * v[j, g]
    return out.reshape(T, H * d) @ W["o"].T


def delta_rule(h, m, W, eps):
    """Per head a state S [key channel, value channel]:
    S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,  o_t = S_t^T r_t."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = (h @ W["r"].T).reshape(T, H, d)
    k = (h @ W["k"].T).reshape(T, H, d)
    v = (h @ W["v"].T).reshape(T, H, d)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ W["w1"].T) @ W["w2"].T + W["w0"])).reshape(T, H, d)
    a = torch.sigmoid(h @ W["a"].T + W["a.b"]).reshape(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d, dtype=F)
    o = torch.zeros(T, H, d, dtype=F)
    for t in range(T):
        for hh in range(H):
            old = S[hh]
            S[hh] = w[t, hh][:, None] * old - torch.outer(a[t, hh] * u[t, hh], u[t, hh] @ old) + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S[hh].T @ r[t, hh]
    o = rms(o, eps).reshape(T, H * d) * W["norm"] * torch.sigmoid(h @ W["g"].T)
    return o @ W["o"].T


def parallel(h, m, W, eps):
    left = sigmoid_attention(h, m["left"], sub(W, "left."), eps)
    right = delta_rule(h, m["right"], sub(W, "right."), eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h, W):
    return (gelu_tanh(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def sub(sd, prefix):
    return {k[len(prefix):]: v for k, v in sd.items() if k.startswith(prefix)}


def forward(cfg, sd, tokens, layers_out=None):
    """Logits [T, vocab] of a whole sequence; ``layers_out``: a list that receives the residual
    stream after every layer."""
    sd = {k: v.to(F) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x = sd["embed"][torch.as_tensor(list(tokens))]
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        W = sub(sd, p + "mix.")
        h = input_conv(x, sd[p + "canon1"])
        if layer["type"] == "latent_attention":
            if "kv_from" in m and m["kv_from"] is not None:
                y = latent_attention(h, m, W, eps, latents[m["kv_from"]])
            else:
                latents[i] = latent_kv(h, m, W, eps)
                y = latent_attention(h, m, W, eps, latents[i])
        elif layer["type"] == "parallel":
            y = parallel(h, m, W, eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms(y, eps) * (1 + sd[p + "norm1"])
        if layer["mlp"] is not None:
            h = input_conv(x, sd[p + "canon2"])
            x = x + rms(dense_ff(h, sub(sd, p + "mlp.")), eps) * (1 + sd[p + "norm2"])
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rms(x, eps) * (1 + sd["final.norm"])
    return h @ sd["head"].T
