"""PyTorch implementations of the sequence-mixer / MoE ops (the CPU backend of
:mod:`.mixers`, and the semantics the HIP kernels in ``csrc/mixers`` must match).

Everything that the kernels keep in fp32 is fp32 here as well: the residual stream,
norm statistics, rotary angles, attention scores and weights, the recurrent state and
all gates and decays that enter the recurrence.  Outputs that feed a matrix product
are rounded once to the requested storage dtype.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def embed_rows(ids, table, scale=1.0, positions=None, pos_freqs=None):
    x = table.index_select(0, ids.long()).float()
    x = x * scale if scale != 1.0 else x
    if pos_freqs is not None:
        x = x + sinusoid_rows(positions[:ids.shape[0]], pos_freqs, x.shape[1])
    return x


def sinusoid_freqs(width: int, base: float = 10000.0, device=None):
    """fp32 [ceil(width / 2)]: f_i = base^(-2i/width), evaluated in double precision."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / width)).float().to(device)


def sinusoid_rows(positions, freqs, width: int):
    """fp32 [T, width]: column 2i = sin(p f_i), column 2i+1 = cos(p f_i) (fp32 angles)."""
    a = positions.float()[:, None] * freqs.float()[None]
    return torch.stack([a.sin(), a.cos()], -1).reshape(positions.shape[0], -1)[:, :width]


def _layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w.float() + b.float()


def layer_norm_rows(x, w, b, eps, out_dtype):
    return _layer_norm(x.float(), w, b, eps).to(out_dtype)


def add_layer_norm_rows(residual, y, w, b, eps, out_dtype):
    if y is None:
        residual.copy_(_layer_norm(residual, w, b, eps))
    else:
        residual.add_(_layer_norm(y.float(), w, b, eps))
    return residual if out_dtype == torch.float32 else residual.to(out_dtype)


def tanh_cap_(x, cap: float):
    """x <- cap * tanh(x / cap) in place (fp32); infinite entries (masked columns) stay."""
    fin = torch.isfinite(x)
    x.copy_(torch.where(fin, cap * torch.tanh(x / cap), x))
    return x


def _rms(x, eps):
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm_rows(x, w, eps, out_dtype, add_vec=None):
    if add_vec is not None:
        x.add_(add_vec.float())
    return (_rms(x, eps) * w.float()).to(out_dtype)


def add_rms_norm_rows(residual, y, wb, eps, add_vec, next_w, out_dtype, want_cast):
    residual.add_(_rms(y.float(), eps) * wb.float())
    if add_vec is not None:
        residual.add_(add_vec.float())
    out = (_rms(residual, eps) * next_w.float()).to(out_dtype) if next_w is not None else None
    cast = residual.to(out_dtype) if want_cast else None
    return out, cast


def add_scaled_rms_norm_rows(residual, y1, y2, mult, next_w, eps, out_dtype):
    if y1 is not None:
        y = y1.float() if y2 is None else y1.float() + y2.float()
        residual.add_(y * mult)
    return (_rms(residual, eps) * next_w.float()).to(out_dtype) if next_w is not None else None


def dual_rms_mean(a, b, wa, wb, eps, scale):
    return scale * (_rms(a.float(), eps) * wa.float() + _rms(b.float(), eps) * wb.float())


def pair_embed_add(x, ids, table, mul_prev: int, mul_cur: int, buckets: int, seg, last_tok):
    start = seg.start.tolist()
    tab = table.float()
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        slot = int(seg.slot[s])
        if b == a or slot < 0:
            continue
        cur = ids[a:b].long()
        first = torch.full((1,), -1, dtype=torch.long) if int(seg.pos0[s]) <= 0 else last_tok[slot].long().view(1)
        prev = torch.cat([first.to(cur.device), cur[:-1]])
        rows = torch.where(prev < 0, torch.full_like(cur, buckets), (prev * mul_prev + cur * mul_cur) % buckets)
        x[a:b] += tab[rows]
        last_tok[slot] = cur[-1].to(last_tok.dtype)
    return x


def sigmoid_gate(o, g, out_dtype):
    return (o.float() * torch.sigmoid(g.float())).to(out_dtype)


def scale_frequencies(f, factor: float, low: float, high: float, original: float):
    """Rotary frequencies stretched for long contexts.  With t_i = original * f_i / (2 pi)
    (how many turns pair i makes over ``original`` positions): f_i stays for t_i > high,
    becomes f_i / factor for t_i < low, and for low <= t_i <= high is the mix
    (1 - s) f_i / factor + s f_i with s = (t_i - low) / (high - low)."""
    wl = 2.0 * math.pi / f
    s = ((original / wl - low) / (high - low)).clamp(0.0, 1.0)
    mid = (1.0 - s) * f / factor + s * f
    return torch.where(wl < original / high, f, torch.where(wl > original / low, f / factor, mid))


def ramp_frequencies(dims: int, base: float, factor: float, original: float, fast: float, slow: float):
    """Rotary frequencies divided by ``factor`` along a linear ramp over the pair index,
    and the factor that goes with them on cos and sin.  With
    where(t) = dims ln(original / (2 pi t)) / (2 ln base) -- the (fractional) pair index
    that makes t turns over ``original`` positions -- lo = max(floor(where(fast)), 0),
    hi = min(ceil(where(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):
    f_i' = r_i f_i / factor + (1 - r_i) f_i; cos and sin are multiplied by
    0.1 ln(factor) + 1.  Evaluated in double precision on the host; returns (fp32 [dims/2],
    float)."""
    where = lambda t: dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))   # noqa: E731
    lo = max(math.floor(where(fast)), 0)
    hi = min(math.ceil(where(slow)), dims - 1)
    f = []
    for i in range(dims // 2):
        fi = float(base) ** (-2.0 * i / dims)
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        f.append(fi / factor * r + fi * (1.0 - r))
    return torch.tensor(f, dtype=torch.float64).to(torch.float32), 0.1 * math.log(factor) + 1.0


def rope_table(max_pos: int, dims: int, base: float, device=None, scaling=None, ramp=None):
    """fp32 [max_pos, dims] = [cos | sin]; frequencies, angles and their cos / sin are
    all evaluated in fp32 (angle = float(p) * f_i, f_i = base^(-2i/dims));
    ``scaling``: (factor, low, high, original) for :func:`scale_frequencies`; ``ramp``:
    (factor, original, fast, slow) for :func:`ramp_frequencies`, whose factor on cos and
    sin is folded into the table."""
    i = torch.arange(dims // 2, dtype=torch.float32)
    f = torch.tensor(float(base), dtype=torch.float32) ** (-2.0 * i / dims)
    mult = 1.0
    if scaling is not None:
        f = scale_frequencies(f, *[float(v) for v in scaling])
    if ramp is not None:
        f, mult = ramp_frequencies(dims, float(base), *[float(v) for v in ramp])
    a = torch.arange(max_pos, dtype=torch.float32)[:, None] * f[None]
    t = torch.cat([a.cos(), a.sin()], -1)
    if mult != 1.0:
        t = t * torch.tensor(mult, dtype=torch.float32)
    return t.to(device)


def distance_bias_table(rel, reach: int):
    """fp32 [reach + 1, heads]: row n is the row of ``rel`` [B, heads] that distance n falls
    into -- n itself below B // 2, then logarithmic steps up to ``reach``:
    min(B - 1, B//2 + floor(ln(n / (B//2)) / ln(reach / (B//2)) (B - B//2))).  Every distance
    of ``reach`` or more falls into the last row, so a kernel clamps the distance to
    ``reach`` and reads this table.  The steps are evaluated in double precision."""
    B = rel.shape[0]
    half = B // 2
    if reach <= half or half < 1:
        raise ValueError("the distance bias needs 1 <= rows // 2 < reach")
    idx = [n if n < half else min(B - 1, half + math.floor(math.log(n / half) / math.log(reach / half) * (B - half)))
           for n in range(reach + 1)]
    return rel.float()[torch.tensor(idx, dtype=torch.long, device=rel.device)].contiguous()


def _rope(x, cs, dims):
    """x [..., T, n] fp32 with cs [T, dims]; rotates the first ``dims`` of n."""
    half = dims // 2
    cos, sin = cs[:, :half], cs[:, half:]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


def short_conv_silu(x, conv_w, conv_state, seg, bias=None):
    t, c = x.shape
    taps = conv_w.shape[1]
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    w = conv_w.float()
    start = seg.start.tolist()
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        slot = int(seg.slot[s])
        if slot < 0 or b == a:
            out[a:b] = 0
            continue
        hist = conv_state[slot] if int(seg.pos0[s]) > 0 else torch.zeros_like(conv_state[slot])
        xp = torch.cat([hist, x[a:b].float()], 0)            # [taps-1 + n, C]
        n = b - a
        y = sum(xp[j:j + n] * w[:, j][None] for j in range(taps))
        if bias is not None:
            y = y + bias.float()
        out[a:b] = (y * torch.sigmoid(y)).to(x.dtype)
        if taps > 1:
            conv_state[slot] = xp[n:]
    return out


def gated_delta_rule(qkv, a, b, a_log, dt_bias, state, seg, heads, kv_heads, dk, dv):
    t = qkv.shape[0]
    rep = heads // kv_heads
    nq = kv_heads * dk
    q = qkv[:, :nq].float().view(t, kv_heads, dk)
    k = qkv[:, nq:2 * nq].float().view(t, kv_heads, dk)
    v = qkv[:, 2 * nq:].float().view(t, heads, dv)
    q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(b.float())
    g = torch.exp(-torch.exp(a_log.float())[None, :, None]
                  * F.softplus(a.float().view(t, heads, dk) + dt_bias.float().view(heads, dk)))
    o = torch.zeros(t, heads, dv, dtype=torch.float32, device=qkv.device)
    start = seg.start.tolist()
    for s in range(seg.num):
        slot = int(seg.slot[s])
        if slot < 0:
            continue
        S = state[slot] if int(seg.pos0[s]) > 0 else torch.zeros_like(state[slot])
        for r in range(start[s], start[s + 1]):
            qt = q[r].repeat_interleave(rep, 0)
            kt = k[r].repeat_interleave(rep, 0)
            S = g[r][:, :, None] * S
            u = beta[r][:, None] * (v[r] - torch.einsum("hkv,hk->hv", S, kt))
            S = S + kt[:, :, None] * u[:, None, :]
            o[r] = torch.einsum("hkv,hk->hv", S, qt)
        state[slot] = S
    return o.view(t, heads * dv)


def gated_linear_attention(qkv, a, a_bias, tau, state, seg, heads, dk, dv):
    t = qkv.shape[0]
    n = heads * dk
    q = qkv[:, :n].float().view(t, heads, dk) * torch.tensor(float(dk), dtype=torch.float32) ** -0.5
    k = qkv[:, n:2 * n].float().view(t, heads, dk)
    v = qkv[:, 2 * n:2 * n + heads * dv].float().view(t, heads, dv)
    g = torch.exp(F.logsigmoid(a.float() + a_bias.float()) / float(tau)).view(t, heads, dk)
    o = torch.zeros(t, heads, dv, dtype=torch.float32, device=qkv.device)
    start = seg.start.tolist()
    for s in range(seg.num):
        slot = int(seg.slot[s])
        if slot < 0:
            continue
        S = state[slot] if int(seg.pos0[s]) > 0 else torch.zeros_like(state[slot])
        for r in range(start[s], start[s + 1]):
            S = g[r][:, :, None] * S + k[r][:, :, None] * v[r][:, None, :]
            o[r] = torch.einsum("hkv,hk->hv", S, q[r])
        if start[s + 1] > start[s]:
            state[slot] = S
    return o.view(t, heads * dv)


def head_rms_gate(o, w, gate_pre, eps, heads, dv, out_dtype, silu=False):
    t = o.shape[0]
    x = o.view(t, heads, dv)
    g = gate_pre.float().reshape(t, heads, dv)
    y = _rms(x, eps) * w.float() * (g * torch.sigmoid(g) if silu else torch.sigmoid(g))
    return y.view(t, heads * dv).to(out_dtype)


def latent_kv_write(dkv, norm_w, eps, table, rot_dims, positions, slot_mapping, cache, rank):
    t = dkv.shape[0]
    if t == 0:
        return
    x = dkv.float()
    c = _rms(x[:, :rank], eps) * norm_w.float()
    kr = _rope(x[:, rank:], table[positions.long()], rot_dims)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    slots = slot_mapping[:t].long()
    keep = slots >= 0
    if keep.any():
        cache.view(-1, cache.shape[-1])[slots[keep]] = row[keep]


def latent_q_rope(q, table, rot_dims, positions, heads, dn, dr):
    """q [T, heads*(dn+dr)] -> (q_unrotated fp32 [T, heads, dn], q_rotated fp32 [T, heads, dr])."""
    t = q.shape[0]
    x = q.float().view(t, heads, dn + dr)
    cs = table[positions.long()]
    return x[..., :dn].contiguous(), _rope(x[..., dn:].transpose(0, 1), cs, rot_dims).transpose(0, 1).contiguous()


def latent_attention(qa, qr, cache, seg, scale, rank):
    """qa fp32 [heads, T, rank] (queries in latent space) and qr fp32 [T, heads, dr]
    (rotated part) against cache rows [c (rank) | rotated key (dr)]; returns the
    softmax-weighted sums of the c rows, fp32 [heads, T, rank]."""
    heads, t, _ = qa.shape
    out = torch.zeros(heads, t, rank, dtype=torch.float32, device=qa.device)
    bs = cache.shape[1]
    start = seg.start.tolist()
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        n = int(seg.kv_len[s])
        if b == a or n == 0:
            continue
        nblk = (n + bs - 1) // bs
        kv = cache[seg.block_tables[s, :nblk].long()].reshape(nblk * bs, -1)[:n].float()
        sc = (torch.einsum("htd,jd->htj", qa[:, a:b], kv[:, :rank])
              + torch.einsum("thd,jd->htj", qr[a:b], kv[:, rank:])) * scale
        qpos = int(seg.pos0[s]) + torch.arange(b - a, device=qa.device)
        mask = torch.arange(n, device=qa.device)[None, :] <= qpos[:, None]
        sc = sc.masked_fill(~mask[None], float("-inf"))
        p = torch.softmax(sc, -1)
        out[:, a:b] = torch.einsum("htj,jr->htr", p, kv[:, :rank])
    return out


def causal_softmax(s, rows_per_head, first_pos, scale, out_dtype):
    rows, keys = s.shape
    qpos = first_pos + torch.arange(rows, device=s.device) % rows_per_head
    mask = torch.arange(keys, device=s.device)[None, :] <= qpos[:, None]
    p = torch.softmax((s.float() * scale).masked_fill(~mask, float("-inf")), -1)
    return p.masked_fill(~mask, 0.0).to(out_dtype)


def moe_topk(z, correction, top, groups, keep):
    s = torch.softmax(z.float(), -1)
    ch = s + correction.float()
    e = z.shape[1]
    if groups > 1 and keep < groups:
        gs = ch.view(-1, groups, e // groups).max(-1).values
        kg = gs.topk(keep, -1).indices
        gm = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, kg, True)
        ch = ch.masked_fill(~gm.repeat_interleave(e // groups, 1), float("-inf"))
    idx = ch.topk(top, -1).indices
    return idx.int(), s.gather(1, idx)


def moe_top_logits(z, top):
    """The ``top`` largest logits per row (ties to the lower index) and the softmax over
    just those."""
    val, idx = torch.sort(z.float(), dim=-1, descending=True, stable=True)
    return idx[:, :top].int(), torch.softmax(val[:, :top], -1)


def moe_pairs(out, h, idx, wts, wgu, wdown, limit, act="clamp_glu"):
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            e = int(idx[t, k])
            u = F.linear(h[t:t + 1], wgu[e])
            y = clamp_swiglu(u, limit) if act == "clamp_glu" else relu_sq(u)
            out[t] += wts[t, k] * F.linear(y, wdown[e])[0].float()


def clamp_swiglu(gu, limit, rows_scale=None):
    """gu [n, 2*ff (+1)] = [gate | up (| per-row gate logit)] -> y [n, ff]:
    g = min(gate, limit), u = clamp(up, +-limit), y = g * sigmoid(1.702 g) * (u + 1)."""
    ff = gu.shape[1] // 2
    g = gu[:, :ff].float().clamp(max=limit)
    u = gu[:, ff:2 * ff].float().clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)).to(gu.dtype)


def relu_sq(x):
    r = torch.relu(x.float())
    return (r * r).to(x.dtype)


def relu_sq_rows(u, ff):
    r = torch.relu(u[:, :ff].float())
    return (r * r).to(u.dtype)


def gather_add_rows(out, y, idx, w):
    out.add_((y.float()[idx.long()] * w.float()[:, :, None]).sum(1))


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z * z * z)))


def side_gate(gpre, table, ids, col0, sd):
    e = table.index_select(0, ids.long())[:, col0:col0 + sd].float()
    return (gelu_tanh(gpre.float()) * e).to(gpre.dtype)


def scale_add_rows(out, y, rows, weights, sigmoid: bool):
    w = weights.float()
    if sigmoid:
        w = torch.sigmoid(w)
    upd = y.float() * w[:, None]
    if rows is None:
        out.add_(upd)
    else:
        out.index_add_(0, rows.long(), upd)


# ---------------------------------------------------------------------------------
# windowed attention over a paged key / value cache, selective state space scan
# ---------------------------------------------------------------------------------

def attn_prep(qkv, nq, nk, q_norm_w, k_norm_w, eps, table, rot_dims, head_dim, positions, slot_mapping,
              k_cache, v_cache):
    t = qkv.shape[0]
    x = qkv.float()
    q, k, v = x[:, :nq], x[:, nq:nq + nk], x[:, nq + nk:]
    if q_norm_w is not None:
        q = _rms(q, eps) * q_norm_w.float()
    if k_norm_w is not None:
        k = _rms(k, eps) * k_norm_w.float()
    if table is not None and rot_dims > 0:
        cs = table[positions[:t].long()]
        q = _rope(q.reshape(t, -1, head_dim).transpose(0, 1), cs, rot_dims).transpose(0, 1).reshape(t, nq)
        k = _rope(k.reshape(t, -1, head_dim).transpose(0, 1), cs, rot_dims).transpose(0, 1).reshape(t, nk)
    if k_cache is None:
        return q.contiguous()
    slots = slot_mapping[:t].long()
    keep = slots >= 0
    if keep.any():
        k_cache.view(-1, k_cache.shape[-1])[slots[keep]] = k[keep].to(k_cache.dtype)
        v_cache.view(-1, v_cache.shape[-1])[slots[keep]] = v[keep].to(v_cache.dtype)
    return q.contiguous()


def conv_attn_prep(qkv, nq, nk, conv_w, conv_state, seg, q_norm_w, k_norm_w, eps, head_dim, slot_mapping,
                   k_cache, v_cache):
    t = qkv.shape[0]
    taps = conv_w.shape[1]
    w = conv_w.float()
    y = torch.zeros(qkv.shape, dtype=torch.float32, device=qkv.device)
    start = seg.start.tolist()
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        slot = int(seg.slot[s])
        if slot < 0 or b == a:
            continue
        hist = conv_state[slot] if int(seg.pos0[s]) > 0 else torch.zeros_like(conv_state[slot])
        xp = torch.cat([hist, qkv[a:b].float()], 0)
        n = b - a
        y[a:b] = sum(xp[j:j + n] * w[:, j][None] for j in range(taps))
        if taps > 1:
            conv_state[slot] = xp[n:]
    q, k, v = y[:, :nq], y[:, nq:nq + nk], y[:, nq + nk:]
    if q_norm_w is not None:
        q = (_rms(q.reshape(t, -1, head_dim), eps) * q_norm_w.float()).reshape(t, nq)
    if k_norm_w is not None:
        k = (_rms(k.reshape(t, -1, head_dim), eps) * k_norm_w.float()).reshape(t, nk)
    slots = slot_mapping[:t].long()
    keep = slots >= 0
    if keep.any():
        k_cache.view(-1, k_cache.shape[-1])[slots[keep]] = k[keep].to(k_cache.dtype)
        v_cache.view(-1, v_cache.shape[-1])[slots[keep]] = v[keep].to(v_cache.dtype)
    return q.contiguous()


def mask_first_key(i: int, window: int, blocks: bool) -> int:
    """The first position that position i sees through its window (or its block)."""
    if window <= 0:
        return 0
    return (i // window) * window if blocks else max(0, i - window + 1)


def band_weights(s, first_pos, key0, window, scale, sigmoid, r1, r2, pb, softcap=0.0, sink=None,
                 blocks=False, keep_first=0, ext=0, dist_bias=None):
    """s fp32 [heads, rows, keys] raw dot products -> attention weights: row r is position
    i = first_pos + r; the first ``ext`` columns are positions 0 .. ext-1 and column
    c >= ext is position j = key0 + c - ext.  Visible iff j <= i and (i - j < window, or
    with ``blocks`` floor(i / window) = floor(j / window), or j < keep_first); window 0:
    every earlier key.  ``dist_bias`` fp32 [nd, heads] adds dist_bias[min(i - j, nd - 1), h]."""
    heads, rows, keys = s.shape
    col = torch.arange(keys, device=s.device)
    jpos = torch.where(col < ext, col, key0 + col - ext)
    ipos = first_pos + torch.arange(rows, device=s.device)
    dist = ipos[:, None] - jpos[None, :]
    vis = dist >= 0
    if window > 0:
        inside = (ipos[:, None] // window == jpos[None, :] // window) if blocks else dist < window
        if keep_first > 0:
            inside = inside | (jpos[None, :] < keep_first)
        vis = vis & inside
    z = s * scale
    if softcap:
        z = softcap * torch.tanh(z / softcap)
    if r1 is not None:
        z = z - r1.float()[:, None, None] * torch.log(1.0 + r2.float()[:, None, None]
                                                      * dist.clamp_min(0).float()[None])
    if dist_bias is not None:
        z = z + dist_bias.float()[dist.clamp(0, dist_bias.shape[0] - 1)].permute(2, 0, 1)
    if sigmoid:
        if pb is not None:
            z = z + pb.float()[:, None, None]
        return torch.sigmoid(z) * vis[None]
    z = z.masked_fill(~vis[None], float("-inf"))
    if sink is not None:
        m = z.max(-1, keepdim=True).values.clamp_min(float(sink))
        e = torch.exp(z - m)
        return e / (torch.exp(float(sink) - m) + e.sum(-1, keepdim=True))
    return torch.softmax(z, -1).masked_fill(~vis[None], 0.0)


def window_attention(q, k_cache, v_cache, seg, heads, maps, kv_heads, dk, dv, window, scale, sigmoid,
                     r1, r2, pb, softcap=0.0, sink=None, blocks=False, keep_first=0, dist_bias=None):
    """q fp32 [T, heads*maps*dk]; caches [blocks, bs, kv_heads*maps*dk] / [blocks, bs,
    kv_heads*dv]; returns fp32 [T, heads*maps, dv]."""
    t = q.shape[0]
    hq = heads * maps
    rep = heads // kv_heads
    out = torch.zeros(t, hq, dv, dtype=torch.float32, device=q.device)
    bs = k_cache.shape[1]
    start = seg.start.tolist()
    a_idx = torch.arange(hq)
    khead = (a_idx // maps // rep) * maps + a_idx % maps
    vhead = a_idx // maps // rep
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        n = int(seg.kv_len[s])
        if b == a or n == 0:
            continue
        p0 = int(seg.pos0[s])
        lo = mask_first_key(p0, window, blocks)
        ext = min(keep_first, lo) if window > 0 else 0
        nblk = (n + bs - 1) // bs
        pages = seg.block_tables[s, :nblk].long()
        keys = torch.cat([torch.arange(ext), torch.arange(lo, n)]).to(k_cache.device)
        k = k_cache[pages].reshape(nblk * bs, -1)[keys].float().view(keys.numel(), kv_heads * maps, dk)
        v = v_cache[pages].reshape(nblk * bs, -1)[keys].float().view(keys.numel(), kv_heads, dv)
        qs = q[a:b].view(b - a, hq, dk)
        sc = torch.einsum("thd,jhd->htj", qs, k[:, khead])
        w = band_weights(sc, p0, lo, window, scale, sigmoid, r1, r2, pb, softcap, sink, blocks, keep_first, ext,
                         dist_bias)
        out[a:b] = torch.einsum("htj,jhd->thd", w, v[:, vhead])
    return out


def diff_combine(a, gate, lam, post_scale, eps, heads, dv, out_dtype):
    t = a.shape[0]
    x = a.view(t, heads, 2, dv)
    o = x[:, :, 0] - lam * x[:, :, 1]
    o = _rms(o, eps) * post_scale * torch.sigmoid(gate.float())[:, :, None]
    return o.reshape(t, heads * dv).to(out_dtype)


def ssd_scan(xbc, dt, a_log, dt_bias, d_skip, state, seg, heads, groups, n, dv):
    t = xbc.shape[0]
    inner = heads * dv
    f = xbc.float()
    x = f[:, :inner].view(t, heads, dv)
    bm = f[:, inner:inner + groups * n].view(t, groups, n)
    cm = f[:, inner + groups * n:].view(t, groups, n)
    step = F.softplus(dt.float() + dt_bias.float(), threshold=1e9)
    decay = torch.exp(-torch.exp(a_log.float())[None] * step)
    grp = torch.arange(heads) // (heads // groups)
    y = torch.zeros(t, heads, dv, dtype=torch.float32, device=xbc.device)
    start = seg.start.tolist()
    for s in range(seg.num):
        slot = int(seg.slot[s])
        if slot < 0:
            continue
        S = state[slot] if int(seg.pos0[s]) > 0 else torch.zeros_like(state[slot])
        for r in range(start[s], start[s + 1]):
            S = decay[r][:, None, None] * S + (step[r][:, None] * bm[r, grp])[:, :, None] * x[r][:, None, :]
            y[r] = (S * cm[r, grp][:, :, None]).sum(1) + d_skip.float()[:, None] * x[r]
        state[slot] = S
    return y.view(t, inner)


def gate_group_norm(y, z, w, eps, groups, out_dtype):
    t, inner = y.shape
    zf = z.float()
    v = y * (zf * torch.sigmoid(zf))
    v = _rms(v.view(t, groups, inner // groups), eps).view(t, inner) * w.float()
    return v.to(out_dtype)


def relu_glu(gu):
    ff = gu.shape[1] // 2
    return (torch.relu(gu[:, :ff].float()) * gu[:, ff:].float()).to(gu.dtype)


def gelu_glu(gu):
    ff = gu.shape[1] // 2
    return (gelu_tanh(gu[:, :ff].float()) * gu[:, ff:].float()).to(gu.dtype)
