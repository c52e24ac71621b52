"""A plain, slow fp32 implementation of the Kerarax design, written from its equations:
one function per mechanism, whole sequences only, no cache, no batching, no package code.

Notation.  ``cfg`` is the configuration as a dict (vocab, width, norm.eps,
logit_softcap, layers[].type / mixer / mlp); ``P`` maps tensor names to fp32 tensors.
x is the residual [T, width]; rows are positions 0 .. T-1 of one sequence.
"""
import math

import torch


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sinusoid(T, width, first=0):
    """[T, width]: column 2i = sin(p f_i), column 2i+1 = cos(p f_i), f_i = 10000^(-2i/width)."""
    out = torch.zeros(T, width)
    for i in range((width + 1) // 2):
        f = 10000.0 ** (-2.0 * i / width)
        for t in range(T):
            a = (first + t) * f
            out[t, 2 * i] = math.sin(a)
            if 2 * i + 1 < width:
                out[t, 2 * i + 1] = math.cos(a)
    return out


def embed(cfg, P, tokens):
    x = P["embed"][torch.tensor(tokens)] + sinusoid(len(tokens), cfg["width"])
    return layer_norm(x, P["embed.norm"], P["embed.norm.b"], cfg["norm"]["eps"])


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before t = 0."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros(T, C)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def capped(s, cap):
    return cap * torch.tanh(s / cap) if cap else s


def sink_softmax(s):
    """Weights exp(s_j) / (1 + sum_j exp(s_j)) over the last axis (-inf entries get 0)."""
    m = s.max(-1, keepdim=True).values.clamp_min(0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attention(m, P, p, h, eps):
    """GQA with short convolutions on q, k, v, per-head RMS norm of q and k, capped scores
    and a softmax whose denominator carries one extra unit (a key of score 0 and no value)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv(h @ P[p + "q"].T, P[p + "q.conv"]).view(T, H, dk)
    k = causal_conv(h @ P[p + "k"].T, P[p + "k.conv"]).view(T, G, dk)
    v = causal_conv(h @ P[p + "v"].T, P[p + "v.conv"]).view(T, G, dv)
    q = rms_unit(q, eps) * P[p + "q.norm"]
    k = rms_unit(k, eps) * P[p + "k.norm"]
    out = torch.zeros(T, H, dv)
    rep = H // G
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for a in range(H):
        g = a // rep
        s = capped((q[:, a] @ k[:, g].T) * m["scale"], m.get("softcap"))
        s = s.masked_fill(~mask, float("-inf"))
        out[:, a] = sink_softmax(s) @ v[:, g]
    return out.reshape(T, H * dv) @ P[p + "o"].T


def expert(P, p, h):
    r = torch.relu(h @ P[p + "up"].T)
    return (r * r) @ P[p + "down"].T


def route(z, top):
    """The ``top`` largest logits of every row and the softmax over just those."""
    val, idx = z.topk(top, -1)
    return idx, torch.softmax(val, -1)


def moe(mlp, P, p, h):
    z = h @ P[p + "router"].T + P[p + "router.b"]
    idx, w = route(z, mlp["router"]["top"])
    y = torch.zeros(h.shape[0], P[p + "e0.down"].shape[0])
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            y[t] += w[t, j] * expert(P, f"{p}e{int(idx[t, j])}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        y = y + torch.sigmoid(h @ P[p + "shared.sg"].T) * expert(P, p + "shared.", h)
    return y


def layers(cfg, P, tokens):
    """The residual after the embedding step and after every layer: list of [T, width]."""
    eps = cfg["norm"]["eps"]
    x = embed(cfg, P, tokens)
    out = []
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        if l["type"] != "attention":
            raise ValueError(l["type"])
        x = x + layer_norm(attention(l["mixer"], P, p + "mix.", x, eps), P[p + "norm1"], P[p + "norm1.b"], eps)
        if l.get("mlp"):
            x = x + layer_norm(moe(l["mlp"], P, p + "mlp.", x), P[p + "norm2"], P[p + "norm2.b"], eps)
        out.append(x)
    return out


def forward(cfg, P, tokens):
    """Logits [T, vocab] of one sequence."""
    x = layers(cfg, P, tokens)[-1] if cfg["layers"] else embed(cfg, P, tokens)
    x = layer_norm(x, P["final.norm"], P["final.norm.b"], cfg["norm"]["eps"])
    return capped(x @ P["head"].T, cfg.get("logit_softcap"))
