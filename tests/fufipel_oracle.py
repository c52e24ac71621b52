"""Plain, slow implementation of the Fufipel design, written from its equations: one
function per mechanism, whole sequences at a time, no cache, no package code.

A model is (cfg, tensors): ``cfg`` the parsed ``config.json`` dict, ``tensors`` a dict of
torch tensors by checkpoint name.  Everything is evaluated in ``DT`` (float64 by default,
so that the comparison's error is the framework's alone).

Notation: T tokens, x the residual [T, width], p = 0..T-1 the positions.
"""
import math

import torch

DT = torch.float64


def _t(x):
    return x.to(DT)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def one_plus_norm(x, w, eps):
    """Residual-stream norm: the stored weight is an offset from one."""
    return rms(x, eps) * (1.0 + _t(w))


def embedding(cfg, ten, tokens):
    """Scaled token row plus an unscaled row of the pair table, chosen by a hash of
    (previous token, token); the first token of a sequence takes the table's last row."""
    e = cfg["embedding"]
    x = _t(ten["embed"])[tokens] * e["scale"]
    bg = e.get("bigram")
    if bg:
        rows = []
        for i, t in enumerate(tokens):
            rows.append(bg["buckets"] if i == 0 else
                        (tokens[i - 1] * bg["mul_prev"] + t * bg["mul_cur"]) % bg["buckets"])
        x = x + _t(ten["bigram"])[rows]
    return x


# ------------------------------------------------------------------------------ positions
def yarn_angles(rot, T):
    """[T, dims/2] angles and the factor on cos and sin."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def where(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(where(sc["fast"])), 0)
        hi = min(math.ceil(where(sc["slow"])), dims - 1)
        out = []
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
        f = out
        mult = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(T, dtype=DT)[:, None] * torch.tensor(f, dtype=DT)[None]
    return ang, mult


def rotate(x, rot):
    """x [T, heads, dim]: the first dims entries of every head, entry i paired with
    i + dims/2."""
    if not rot or not rot.get("dims"):
        return x
    dims = rot["dims"]
    half = dims // 2
    ang, mult = yarn_angles(rot, x.shape[0])
    c, s = (ang.cos() * mult)[:, None, :], (ang.sin() * mult)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# ------------------------------------------------------------------------------ masks
def visible(mask, T, kind):
    """[T, T] bool: row i, column j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = j <= i
    if not mask:
        return vis
    size = mask["size"]
    if kind == "chunk":
        return vis & (i // size == j // size)
    return vis & ((i - j < size) | (j < mask.get("keep_first", 0)))


def distance_bucket(n, B, D):
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + math.floor(math.log(n / half) / math.log(D / half) * (B - half)))


def distance_bias(rel, D, T):
    """[heads, T, T] from the table rel [B, heads]; entries above the diagonal are unused."""
    B = rel.shape[0]
    idx = torch.zeros(T, T, dtype=torch.long)
    for d in range(T):
        b = distance_bucket(d, B, D)
        for i in range(d, T):
            idx[i, i - d] = b
    return _t(rel)[idx].permute(2, 0, 1)


def softmax_attention(q, k, v, scale, vis, bias=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] -> [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[-1], dtype=DT)
    for h in range(H):
        g = h // rep
        s = q[:, h] @ k[:, g].T * scale
        if bias is not None:
            s = s + bias[h]
        s = s.masked_fill(~vis, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


# ------------------------------------------------------------------------------ mixers
def lin(ten, name, h):
    return h @ _t(ten[name]).T


def rope_chunk_attention(cfg, ten, p, m, h):
    """Grouped-query attention with partly rotated heads; a position sees the earlier
    positions of its own block of mask.size positions (blocks counted from 0)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = rotate(lin(ten, p + "q", h).view(T, H, dk), m.get("rot"))
    k = rotate(lin(ten, p + "k", h).view(T, G, dk), m.get("rot"))
    v = lin(ten, p + "v", h).view(T, G, dv)
    o = softmax_attention(q, k, v, m["scale"], visible(m.get("mask"), T, "chunk"))
    return lin(ten, p + "o", o.reshape(T, H * dv))


def gated_linear_attention(cfg, ten, p, m, h):
    """S_t = diag(alpha_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t per head; alpha in (0, 1)
    per key channel."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    eps = cfg["norm"]["eps"]
    q = lin(ten, p + "q", h).view(T, H, dk) * dk ** -0.5
    k = lin(ten, p + "k", h).view(T, H, dk)
    v = lin(ten, p + "v", h).view(T, H, dv)
    z = lin(ten, p + "a2", lin(ten, p + "a1", h)) + _t(ten[p + "a2.b"])
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / m["tau"]).view(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=DT)
    o = torch.zeros(T, H, dv, dtype=DT)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms(o, eps) * _t(ten[p + "norm"])
    g = lin(ten, p + "g", h)
    return lin(ten, p + "o", o.reshape(T, H * dv) * (g * torch.sigmoid(g)))


def side_by_side(cfg, ten, p, m, h):
    eps = cfg["norm"]["eps"]
    a = rope_chunk_attention(cfg, ten, p + "left.", m["left"], h)
    b = gated_linear_attention(cfg, ten, p + "right.", m["right"], h)
    return 0.5 * (rms(a, eps) * _t(ten[p + "left.out"]) + rms(b, eps) * _t(ten[p + "right.out"]))


def keys_values(cfg, ten, p, m, h):
    T = h.shape[0]
    G, dk, dv = m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    k = rms(lin(ten, p + "k", h), cfg["norm"]["eps"]) * _t(ten[p + "k.norm"])
    return k.view(T, G, dk), lin(ten, p + "v", h).view(T, G, dv)


def biased_window_attention(cfg, ten, p, m, h, kv):
    """Grouped-query attention without rotation: q and k normed over the whole projection,
    a bias per head by bucketed distance, a sliding window that also keeps the first
    tokens, and a sigmoid gate on the heads' outputs.  ``kv``: the (k, v) of the layer
    whose keys and values this one reads."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (rms(lin(ten, p + "q", h), cfg["norm"]["eps"]) * _t(ten[p + "q.norm"])).view(T, H, dk)
    k, v = kv
    bias = distance_bias(ten[p + "rel"], m["bias_max"], T)
    o = softmax_attention(q, k, v, m["scale"], visible(m.get("mask"), T, "window"), bias)
    o = o.reshape(T, H * dv) * torch.sigmoid(lin(ten, p + "g", h))
    return lin(ten, p + "o", o)


def feed_forward(ten, p, h):
    return lin(ten, p + "down", torch.relu(lin(ten, p + "gate", h)) * lin(ten, p + "up", h))


# ------------------------------------------------------------------------------ the model
def forward(cfg, ten, tokens, taps=None):
    """Logits [T, vocab]; ``taps`` (a list) receives the residual after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = embedding(cfg, ten, list(tokens))
    kvs = {}
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = one_plus_norm(x, ten[p + "norm1"], eps)
        m = l["mixer"]
        if l["type"] == "parallel":
            y = side_by_side(cfg, ten, p + "mix.", m, h)
        elif l["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = keys_values(cfg, ten, p + "mix.", m, h)
                src = i
            y = biased_window_attention(cfg, ten, p + "mix.", m, h, kvs[src])
        else:
            raise ValueError(l["type"])
        if l.get("mlp"):
            y = y + feed_forward(ten, p + "mlp.", h)
        x = x + mult * y
        if taps is not None:
            taps.append(x.clone())
    h = one_plus_norm(x, ten["final.norm"], eps)
    return h @ _t(ten["embed"]).T * cfg.get("logit_scale", 1.0)


def greedy(cfg, ten, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, ten, toks)[-1].argmax()))
    return toks[len(prompt):]


def layers(cfg, ten, tokens):
    taps = []
    forward(cfg, ten, tokens, taps)
    return taps
