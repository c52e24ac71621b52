"""Sequence-mixer and mixture-of-experts ops: latent (low-rank KV) attention over a
paged latent cache, windowed attention (softmax or sigmoid weights, distance bias,
several score maps per head, capped scores, a sink in the softmax) over a paged key /
value cache, the gated delta-rule recurrence with per-channel decay and the selective
state-space scan over state slots, short causal convolutions (alone, or fused with
per-head norms and the cache write), routing (grouped softmax top-k, or top-k on the
logits), clamped-GLU and relu^2 experts (per-pair kernels for few rows, a grouped product
for many), and the fp32-residual norms (RMS pre/post norms, layer norm with bias) that tie
them together.

GPU tensors run the gfx950 kernels of the ``_C_mixers`` extension (``csrc/mixers``),
fp32 or bf16 activations with fp32 statistics / scores / state; CPU tensors run the
PyTorch implementations in :mod:`.mixers_ref`.  As in :mod:`fasttalk_llm_microservice_amd.ops`
there is no silent fallback for GPU tensors.

A step's rows are described by :class:`Segments`: every scheduled sequence contributes
one segment of consecutive rows (a decode row is a segment of one row, a prefill chunk
a longer one), with the position of its first row, its state slot and its block table.
"""
from __future__ import annotations

import dataclasses
import importlib
import os
import threading
from typing import Optional

import torch

from . import mixers_ref as ref

_lock = threading.Lock()
_M = None


def native_mixers():
    """The loaded ``_C_mixers`` extension, built in-tree on first use if allowed."""
    global _M
    if _M is not None:
        return _M
    with _lock:
        if _M is not None:
            return _M
        try:
            mod = importlib.import_module("fasttalk_llm_microservice_amd._C_mixers")
        except ImportError as e:
            if os.environ.get("FT_AUTOBUILD", "1") == "0":
                raise RuntimeError("fasttalk native extension _C_mixers is not built; run "
                                   "`python -m fasttalk_llm_microservice_amd.ops.build --only mixers`") from e
            from .build import build_mixers

            build_mixers(verbose=True)
            mod = importlib.import_module("fasttalk_llm_microservice_amd._C_mixers")
        _M = mod
        return _M


@dataclasses.dataclass
class Segments:
    """Row segments of one step (device int32 tensors; ``num`` / ``max_rows`` host ints)."""
    start: torch.Tensor          # [num + 1] first row of each segment, then the row count
    pos0: torch.Tensor           # [num] sequence position of the segment's first row
    slot: torch.Tensor           # [num] recurrent-state slot (-1: padding, state untouched)
    kv_len: torch.Tensor         # [num] context length once this step's rows are written
    block_tables: torch.Tensor   # [num, max_blocks]
    num: int
    max_rows: int                # longest segment (rows)
    max_kv: int = 0              # longest context (tokens); 0 = unknown
    # host copies of start / pos0 / kv_len (eager steps; None inside captured graphs)
    host: Optional[tuple] = None


# ---------------------------------------------------------------------------------
# residual stream (fp32) and norms
# ---------------------------------------------------------------------------------

def embed_rows(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0,
               positions: Optional[torch.Tensor] = None,
               pos_freqs: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 residual rows table[ids] * scale; with ``pos_freqs`` (fp32 [ceil(width/2)],
    :func:`sinusoid_freqs`) a sinusoidal position vector is added: column 2i gets
    sin(p f_i), column 2i+1 cos(p f_i), angles in fp32."""
    if ids.is_cuda:
        out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=ids.device)
        native_mixers().embed_rows(out, ids, table, float(scale), positions if pos_freqs is not None else None,
                                   pos_freqs)
        return out
    return ref.embed_rows(ids, table, scale, positions, pos_freqs)


sinusoid_freqs = ref.sinusoid_freqs


def layer_norm_rows(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w + b of fp32 rows x (var = mean squared deviation),
    rounded to ``out_dtype``; x is left as it is."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        native_mixers().layer_norm(x, None, w, b, out, None, eps)
        return out
    return ref.layer_norm_rows(x, w, b, eps, out_dtype)


def add_layer_norm_rows(residual: torch.Tensor, y: Optional[torch.Tensor], w: torch.Tensor, b: torch.Tensor,
                        eps: float, out_dtype) -> torch.Tensor:
    """residual (fp32, in place) += layer_norm(y) * w + b, or, without y, residual <-
    layer_norm(residual) * w + b.  Returns the new residual in ``out_dtype`` (the residual
    itself when that is fp32): what the next sublayer of a post-norm stack reads."""
    if residual.is_cuda:
        cast = None if out_dtype == torch.float32 else \
            torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
        native_mixers().layer_norm(residual, y, w, b, None, cast, eps)
        return residual if cast is None else cast
    return ref.add_layer_norm_rows(residual, y, w, b, eps, out_dtype)


def tanh_cap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """fp32 x <- cap * tanh(x / cap) in place; infinite entries stay as they are."""
    if x.is_cuda:
        native_mixers().tanh_cap(x, float(cap))
        return x
    return ref.tanh_cap_(x, cap)


def rms_norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype,
                  add_vec: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = x / sqrt(mean(x^2) + eps) * w of fp32 rows x, rounded to ``out_dtype``;
    with ``add_vec`` the rows are first updated in place, x += add_vec."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        native_mixers().add_rms_norm(x, None, None, add_vec, w, out, None, eps)
        return out
    return ref.rms_norm_rows(x, w, eps, out_dtype, add_vec)


def add_rms_norm_rows(residual: torch.Tensor, y: torch.Tensor, wb: torch.Tensor, eps: float,
                      add_vec: Optional[torch.Tensor] = None, next_w: Optional[torch.Tensor] = None,
                      out_dtype=None, want_cast: bool = False):
    """residual (fp32, in place) += rms_norm(y) * wb (+ add_vec); returns
    (rms_norm(residual) * next_w or None, residual cast to out_dtype or None)."""
    out_dtype = out_dtype or y.dtype
    if residual.is_cuda:
        out = torch.empty(residual.shape, dtype=out_dtype, device=y.device) if next_w is not None else None
        cast = torch.empty(residual.shape, dtype=out_dtype, device=y.device) if want_cast else None
        native_mixers().add_rms_norm(residual, y, wb, add_vec, next_w, out, cast, eps)
        return out, cast
    return ref.add_rms_norm_rows(residual, y, wb, eps, add_vec, next_w, out_dtype, want_cast)


def add_scaled_rms_norm_rows(residual: torch.Tensor, y1: Optional[torch.Tensor], y2: Optional[torch.Tensor],
                             mult: float, next_w: Optional[torch.Tensor], eps: float, out_dtype):
    """residual (fp32, in place) += mult * (y1 + y2); returns rms_norm(residual) * next_w in
    ``out_dtype`` (None without ``next_w``).  y1 and y2 may be fp32 or bf16 each; y2, or
    both, may be absent (then only the norm is taken).  The step between the layers of a
    stack whose mixer and feed-forward read one shared norm and are added together."""
    if residual.is_cuda:
        out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device) if next_w is not None else None
        native_mixers().add_scaled_rms_norm(residual, y1, y2, float(mult), next_w, out, eps)
        return out
    return ref.add_scaled_rms_norm_rows(residual, y1, y2, mult, next_w, eps, out_dtype)


def dual_rms_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float,
                  scale: float = 0.5) -> torch.Tensor:
    """fp32 scale * (rms_norm(a) * wa + rms_norm(b) * wb) of two rows of equal width: the
    outputs of two mixers that run side by side, each normed on its own."""
    if a.is_cuda:
        out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
        native_mixers().dual_rms_mean(out, a, b, wa, wb, eps, float(scale))
        return out
    return ref.dual_rms_mean(a, b, wa, wb, eps, scale)


def pair_embed_add(x: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, mul_prev: int, mul_cur: int,
                   buckets: int, seg: "Segments", last_tok: torch.Tensor) -> torch.Tensor:
    """x (fp32 rows, in place) += table[(prev * mul_prev + cur * mul_cur) mod buckets], prev
    being the token before the row's own in its sequence; a sequence's first token takes
    row ``buckets``.  The token before a segment's first row comes from ``last_tok``
    [slots] int32 (the sequence's state slot), which is then set to the segment's last
    token."""
    if x.is_cuda:
        native_mixers().pair_embed_add(x, ids, table, int(mul_prev), int(mul_cur), int(buckets), seg.start,
                                       seg.pos0, seg.slot, seg.num, last_tok, None, 1.0)
        return x
    return ref.pair_embed_add(x, ids, table, mul_prev, mul_cur, buckets, seg, last_tok)


def pair_embed_rows(ids: torch.Tensor, embed: torch.Tensor, scale: float, table: torch.Tensor, mul_prev: int,
                    mul_cur: int, buckets: int, seg: "Segments", last_tok: torch.Tensor) -> torch.Tensor:
    """:func:`embed_rows` and :func:`pair_embed_add` in one launch: fp32 rows
    embed[ids] * scale + table[hash(previous token, token)]."""
    if ids.is_cuda:
        x = torch.empty(ids.shape[0], embed.shape[1], dtype=torch.float32, device=ids.device)
        native_mixers().pair_embed_add(x, ids, table, int(mul_prev), int(mul_cur), int(buckets), seg.start,
                                       seg.pos0, seg.slot, seg.num, last_tok, embed, float(scale))
        return x
    return ref.pair_embed_add(ref.embed_rows(ids, embed, scale), ids, table, mul_prev, mul_cur, buckets, seg, last_tok)


def sigmoid_gate(o: torch.Tensor, g: torch.Tensor, out_dtype) -> torch.Tensor:
    """o * sigmoid(g) element by element (o fp32 [T, n]; g [T, n], may be a column range of
    wider rows), rounded to ``out_dtype``."""
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        native_mixers().sigmoid_gate(out, o, g)
        return out
    return ref.sigmoid_gate(o, g, out_dtype)


# ---------------------------------------------------------------------------------
# rotary positions (partial, rotate-half pairs, fp32 angles)
# ---------------------------------------------------------------------------------

rope_table = ref.rope_table
ramp_frequencies = ref.ramp_frequencies
distance_bias_table = ref.distance_bias_table


# ---------------------------------------------------------------------------------
# short convolution + gated delta rule (recurrent state slots)
# ---------------------------------------------------------------------------------

def short_conv_silu(x: torch.Tensor, conv_w: torch.Tensor, conv_state: torch.Tensor, seg: Segments,
                    bias: Optional[torch.Tensor] = None):
    """Per-channel causal convolution over time (+ ``bias`` [C] fp32), then SiLU.
    ``conv_w`` [C, taps] fp32 (last column = the current row); ``conv_state`` [slots,
    taps-1, C] fp32 holds each sequence's last inputs and is updated; a segment at
    position 0 starts from zeros.  ``x`` may be a column range of wider rows."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        native_mixers().short_conv_silu(out, x, conv_w, bias, conv_state, seg.start, seg.pos0, seg.slot,
                                        seg.num, seg.max_rows)
        return out
    return ref.short_conv_silu(x, conv_w, conv_state, seg, bias)


def gated_delta_rule(qkv, a, b, a_log, dt_bias, state, seg: Segments, heads: int, kv_heads: int,
                     dk: int, dv: int) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel.

    Rows of ``qkv`` are [q (kv_heads*dk) | k (kv_heads*dk) | v (heads*dv)] after the
    short convolution; q and k are unit-normalised per head here (q also * dk^-1/2),
    beta = sigmoid(b), decay = exp(-exp(a_log) * softplus(a + dt_bias)).  Per head and
    row:  S <- decay (.) S (rows of S);  u = beta (v - S^T k);  S <- S + k u^T;
    o = S^T q.  ``state`` [slots, heads, dk, dv] fp32 is read (zeros at position 0)
    and left at the segment's last row.  Returns o fp32 [T, heads*dv]."""
    if qkv.is_cuda:
        o = torch.empty(qkv.shape[0], heads * dv, dtype=torch.float32, device=qkv.device)
        native_mixers().gated_delta_rule(o, qkv, a, b, a_log, dt_bias, state, seg.start, seg.pos0,
                                         seg.slot, seg.num, heads, kv_heads, dk, dv)
        return o
    return ref.gated_delta_rule(qkv, a, b, a_log, dt_bias, state, seg, heads, kv_heads, dk, dv)


def gated_linear_attention(qkv, a, a_bias, tau: float, state, seg: Segments, heads: int, dk: int,
                           dv: int) -> torch.Tensor:
    """Linear attention with a decay per head and key channel.

    Rows of ``qkv`` are [q (heads*dk) | k (heads*dk) | v (heads*dv) | ...]; q is scaled by
    dk^-1/2; decay = sigmoid(a + a_bias)^(1/tau), evaluated as exp(log sigmoid(.) / tau) in
    fp32.  Per head and row:  S <- diag(decay) S + k v^T;  o = S^T q.  ``state`` [slots,
    heads, dk, dv] fp32 is read (zeros at position 0) and left at the segment's last row.
    Returns o fp32 [T, heads*dv]."""
    if qkv.is_cuda:
        o = torch.empty(qkv.shape[0], heads * dv, dtype=torch.float32, device=qkv.device)
        native_mixers().gated_linear_attention(o, qkv, a, a_bias, float(tau), state, seg.start, seg.pos0,
                                               seg.slot, seg.num, seg.max_rows, heads, dk, dv)
        return o
    return ref.gated_linear_attention(qkv, a, a_bias, tau, state, seg, heads, dk, dv)


def head_rms_gate(o, w, gate_pre, eps: float, heads: int, dv: int, out_dtype, silu: bool = False):
    """Per head: o / rms(o) * w * sigmoid(gate_pre) (or * silu(gate_pre)), rounded to
    ``out_dtype``; ``gate_pre`` [T, heads*dv] may be a column range of wider rows."""
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        native_mixers().head_rms_gate(out, o, w, gate_pre, eps, heads, dv, bool(silu))
        return out
    return ref.head_rms_gate(o, w, gate_pre, eps, heads, dv, out_dtype, silu)


# ---------------------------------------------------------------------------------
# latent attention (paged cache of [normed latent | rotated shared key])
# ---------------------------------------------------------------------------------

def latent_kv_write(dkv, norm_w, eps: float, table, rot_dims: int, positions, slot_mapping, cache,
                    rank: int):
    """Cache row = [rms_norm(dkv[:rank]) * norm_w | rope(dkv[rank:])] at each row's slot."""
    if dkv.is_cuda:
        native_mixers().latent_kv_write(dkv, norm_w, eps, table, rot_dims, positions, slot_mapping,
                                        cache, rank)
    else:
        ref.latent_kv_write(dkv, norm_w, eps, table, rot_dims, positions, slot_mapping, cache, rank)


def latent_q_rope(q, table, rot_dims: int, positions, heads: int, dn: int, dr: int):
    """q rows [heads x (dn unrotated | dr rotated)] -> fp32 ([T, heads, dn], [T, heads, dr] rotated)."""
    if q.is_cuda:
        t = q.shape[0]
        qn = torch.empty(t, heads, dn, dtype=torch.float32, device=q.device)
        qr = torch.empty(t, heads, dr, dtype=torch.float32, device=q.device)
        native_mixers().latent_q_rope(qn, qr, q, table, rot_dims, positions, heads, dn, dr)
        return qn, qr
    return ref.latent_q_rope(q, table, rot_dims, positions, heads, dn, dr)


def latent_attention(qa, qr, cache, seg: Segments, scale: float, rank: int,
                     skip_from: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal softmax attention over the paged latent cache.  ``qa`` fp32 [heads, T,
    rank]: the unrotated query parts carried into latent space (q W_uk); ``qr`` fp32
    [T, heads, dr]: the rotated parts.  Score = (qa . c + qr . k_rot) * scale; all heads
    share the cached row, whose first ``rank`` entries are also the value.  Returns
    fp32 [heads, T, rank].  ``skip_from`` > 0: segments of that many rows or more are
    left to the caller (:func:`latent_attention_products`)."""
    if qa.is_cuda:
        if out is None:
            out = torch.empty_like(qa)
        native_mixers().latent_attention(out, qa, qr, cache, seg.start, seg.pos0, seg.kv_len,
                                         seg.block_tables, seg.num, seg.max_rows, scale, rank,
                                         skip_from, seg.max_kv)
        return out
    r = ref.latent_attention(qa, qr, cache, seg, scale, rank)
    if out is not None:
        out.copy_(r)
        return out
    return r


def causal_softmax(s, rows_per_head: int, first_pos: int, scale: float, out_dtype):
    """P = softmax(scale * S) per row over the keys j <= first_pos + (row mod
    rows_per_head), zeros beyond; S fp32 [heads * rows_per_head, keys]."""
    if s.is_cuda:
        p = torch.empty(s.shape, dtype=out_dtype, device=s.device)
        native_mixers().causal_softmax(p, s, rows_per_head, first_pos, scale)
        return p
    return ref.causal_softmax(s, rows_per_head, first_pos, scale, out_dtype)


_MM_F32_OUT = {}


def mm_f32(a, b):
    """a @ b with fp32 accumulation and fp32 output (operands fp32, or bf16 where the
    vendor library returns fp32 from bf16 operands; otherwise widened first)."""
    if a.dtype == torch.float32:
        return torch.mm(a, b)
    ok = _MM_F32_OUT.get(a.device.type)
    if ok is None and a.is_cuda:
        try:
            torch.mm(a[:1], b[:, :1], out_dtype=torch.float32)
            ok = True
        except (TypeError, RuntimeError):
            ok = False
        _MM_F32_OUT[a.device.type] = ok
    return torch.mm(a, b, out_dtype=torch.float32) if ok else torch.mm(a.float(), b.float())


# bytes of fp32 scores the product path holds at once
PRODUCT_SCORE_BYTES = 1 << 30


def latent_attention_products(out, qa, qr, cache, seg: Segments, scale: float, rank: int,
                              min_rows: int, dtype):
    """Segments of ``min_rows`` rows or more as two matrix products: all heads share
    the cached rows, so with M = heads x rows the scores are Q [M, rank+dr] C^T and the
    sums P [M, keys] C[:, :rank], with a causal softmax (fp32 statistics) in between.
    Needs the segments' host copies; writes its rows of ``out`` [heads, T, rank]."""
    start, pos0, kv_len = seg.host
    heads = qa.shape[0]
    bs = cache.shape[1]
    width = cache.shape[2]
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        n = b - a
        if n < min_rows:
            continue
        nblk = (kv_len[s] + bs - 1) // bs
        kv = cache.index_select(0, seg.block_tables[s, :nblk].long()).view(nblk * bs, width)
        step = max(1, min(n, PRODUCT_SCORE_BYTES // (4 * heads * max(1, kv_len[s]))))
        for c0 in range(0, n, step):
            c1 = min(n, c0 + step)
            keys = min(kv_len[s], pos0[s] + c1)          # the chunk's last row sees this many
            q = torch.cat([qa[:, a + c0:a + c1], qr[a + c0:a + c1].transpose(0, 1)], -1) \
                .reshape(heads * (c1 - c0), width).to(dtype)
            sc = mm_f32(q, kv[:keys].t())
            p = causal_softmax(sc, c1 - c0, pos0[s] + c0, scale, dtype)
            out[:, a + c0:a + c1] = mm_f32(p, kv[:keys, :rank]).view(heads, c1 - c0, rank)
    return out


# ---------------------------------------------------------------------------------
# selective state-space scan (recurrent state slots)
# ---------------------------------------------------------------------------------

def ssd_scan(xbc, dt, a_log, dt_bias, d_skip, state, seg: Segments, heads: int, groups: int, n: int,
             dv: int) -> torch.Tensor:
    """State-space recurrence with one scalar decay per head and row.

    Rows of ``xbc`` are [x (heads*dv) | B (groups*n) | C (groups*n)] after the short
    convolution; ``dt`` [T, heads] is the raw step projection (may be a column range).
    step = softplus(dt + dt_bias), decay = exp(-exp(a_log) * step); per head (group
    floor(h / (heads / groups))) and row:  S <- decay S + step B x^T (S is n x dv);
    y = S^T C + d_skip x.  ``state`` [slots, heads, n, dv] fp32 is read (zeros at
    position 0) and left at the segment's last row.  Returns y fp32 [T, heads*dv]."""
    if xbc.is_cuda:
        y = torch.empty(xbc.shape[0], heads * dv, dtype=torch.float32, device=xbc.device)
        native_mixers().ssd_scan(y, xbc, dt, a_log, dt_bias, d_skip, state, seg.start, seg.pos0, seg.slot,
                                 seg.num, heads, groups, n, dv)
        return y
    return ref.ssd_scan(xbc, dt, a_log, dt_bias, d_skip, state, seg, heads, groups, n, dv)


def gate_group_norm(y, z, w, eps: float, groups: int, out_dtype):
    """v = y * silu(z); each of ``groups`` equal parts of a row divided by its own root
    mean square; times w.  y fp32 [T, n], z [T, n] (may be a column range)."""
    if y.is_cuda:
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        native_mixers().gate_group_norm(out, y, z, w, eps, groups)
        return out
    return ref.gate_group_norm(y, z, w, eps, groups, out_dtype)


# ---------------------------------------------------------------------------------
# windowed attention (paged key cache + paged value cache)
# ---------------------------------------------------------------------------------

def attn_prep(qkv, nq: int, nk: int, q_norm_w, k_norm_w, eps: float, table, rot_dims: int,
              head_dim: int, positions, slot_mapping, k_cache, v_cache) -> torch.Tensor:
    """Rows [q (nq) | k (nk) | v] of a fused projection -> fp32 queries [T, nq]; keys and
    values go to the rows' cache slots.  Optional steps, in this order: RMS norm of the
    whole q part and of the whole k part with weights ``q_norm_w`` / ``k_norm_w``; rotary
    positions on the first ``rot_dims`` entries of every ``head_dim`` chunk of q and k
    (entry i paired with i + rot_dims/2, ``table`` = :func:`rope_table`).  Without caches
    (``nk`` 0, rows of q alone) only the queries are prepared."""
    if qkv.is_cuda:
        q = torch.empty(qkv.shape[0], nq, dtype=torch.float32, device=qkv.device)
        native_mixers().attn_prep(q, qkv, nq, nk, q_norm_w, k_norm_w, eps, table, rot_dims, head_dim,
                                  positions, slot_mapping, k_cache, v_cache)
        return q
    return ref.attn_prep(qkv, nq, nk, q_norm_w, k_norm_w, eps, table, rot_dims, head_dim, positions,
                         slot_mapping, k_cache, v_cache)


def conv_attn_prep(qkv, nq: int, nk: int, conv_w, conv_state, seg: Segments, q_norm_w, k_norm_w, eps: float,
                   head_dim: int, slot_mapping, k_cache, v_cache) -> torch.Tensor:
    """Rows [q (nq) | k (nk) | v] of a fused projection pass a per-channel causal
    convolution over time (``conv_w`` [C, taps] fp32, last column = the current row, no
    bias, no activation; ``conv_state`` [slots, taps-1, C] fp32 holds each sequence's last
    projected rows and is updated; a segment at position 0 starts from zeros), then every
    ``head_dim`` chunk of q and of k is divided by its root mean square and multiplied by
    ``q_norm_w`` / ``k_norm_w`` ([head_dim], shared by the heads; None: no norm).
    Convolution and norm are fp32.  Returns fp32 queries [T, nq]; keys and values go to
    the rows' cache slots."""
    if qkv.is_cuda:
        q = torch.empty(qkv.shape[0], nq, dtype=torch.float32, device=qkv.device)
        native_mixers().conv_attn_prep(q, qkv, nq, nk, conv_w, conv_state, seg.start, seg.pos0, seg.slot, seg.num,
                                       q_norm_w, k_norm_w, eps, head_dim, slot_mapping, k_cache, v_cache)
        return q
    return ref.conv_attn_prep(qkv, nq, nk, conv_w, conv_state, seg, q_norm_w, k_norm_w, eps, head_dim,
                              slot_mapping, k_cache, v_cache)


@dataclasses.dataclass
class WindowSpec:
    """A windowed attention's constants.  Query head a = h * maps + m (head h, score map
    m) reads key head floor(h / (heads / kv_heads)) * maps + m and value head
    floor(h / (heads / kv_heads)).  Position i sees j iff 0 <= i - j < window (window 0:
    every earlier key); with ``blocks`` the window is a block instead, j <= i and
    floor(i / window) = floor(j / window), blocks counted from position 0; with
    ``keep_first`` f > 0 the positions j < f stay visible whatever the window.
    s = q.k * scale; with ``softcap`` c > 0, s <- c tanh(s / c);
    score = s - r1[a] ln(1 + r2[a] (i - j)) + dist_bias[min(i - j, nd - 1), a]; weight =
    softmax over the visible keys, or sigmoid(score + pb[a]) without normalisation.
    ``sink`` (a score, softmax only): the softmax's denominator gains exp(sink), as if one
    more key with that score and no value were always visible."""
    heads: int
    kv_heads: int
    dk: int
    dv: int
    window: int
    scale: float
    maps: int = 1
    sigmoid: bool = False
    r1: Optional[torch.Tensor] = None     # fp32 [heads * maps] (with r2)
    r2: Optional[torch.Tensor] = None
    pb: Optional[torch.Tensor] = None     # fp32 [heads * maps] (sigmoid weights only)
    softcap: float = 0.0
    sink: Optional[float] = None
    blocks: bool = False
    keep_first: int = 0
    dist_bias: Optional[torch.Tensor] = None   # fp32 [nd, heads * maps], :func:`distance_bias_table`


def window_attention(q, k_cache, v_cache, seg: Segments, spec: WindowSpec, skip_from: int = 0,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q fp32 [T, heads*maps*dk] against the paged caches; fp32 [T, heads*maps, dv].
    ``skip_from`` > 0: segments of that many rows or more are left to the caller
    (:func:`window_attention_products`)."""
    sp = spec
    if q.is_cuda:
        if out is None:
            out = torch.empty(q.shape[0], sp.heads * sp.maps, sp.dv, dtype=torch.float32, device=q.device)
        native_mixers().window_attention(out, q, k_cache, v_cache, seg.start, seg.pos0, seg.kv_len,
                                         seg.block_tables, seg.num, seg.max_rows, sp.heads, sp.maps,
                                         sp.kv_heads, sp.dk, sp.dv, sp.window, sp.scale, sp.sigmoid,
                                         sp.r1, sp.r2, sp.pb, skip_from, float(sp.softcap), sp.sink,
                                         bool(sp.blocks), int(sp.keep_first), sp.dist_bias)
        return out
    r = ref.window_attention(q, k_cache, v_cache, seg, sp.heads, sp.maps, sp.kv_heads, sp.dk, sp.dv,
                             sp.window, sp.scale, sp.sigmoid, sp.r1, sp.r2, sp.pb, sp.softcap, sp.sink,
                             sp.blocks, sp.keep_first, sp.dist_bias)
    if out is not None:
        out.copy_(r)
        return out
    return r


def band_weights(s, first_pos: int, key0: int, spec: WindowSpec, rep_rows: int, ext: int = 0):
    """Raw dot products fp32 [kv_heads*maps, rep*rows, keys] (the query heads that share
    a key head stacked along the rows, ``rep_rows`` = rows of one of them) -> attention
    weights fp32, in place: row r of a head is position first_pos + r; the first ``ext``
    columns are the positions 0 .. ext-1 (kept first tokens in front of the band), column
    c >= ext is position key0 + c - ext."""
    sp = spec
    if s.is_cuda:
        native_mixers().band_weights(s, rep_rows, first_pos, key0, sp.heads, sp.maps, sp.kv_heads,
                                     sp.window, sp.scale, sp.sigmoid, sp.r1, sp.r2, sp.pb, float(sp.softcap),
                                     sp.sink, bool(sp.blocks), int(sp.keep_first), int(ext), sp.dist_bias)
        return s
    g, rr, keys = s.shape
    rep = sp.heads // sp.kv_heads
    # [G, maps, rep, rows, keys] -> query-head order (g, r, m)
    v = s.view(sp.kv_heads, sp.maps, rep, rep_rows, keys).permute(0, 2, 1, 3, 4) \
        .reshape(sp.heads * sp.maps, rep_rows, keys)
    w = ref.band_weights(v, first_pos, key0, sp.window, sp.scale, sp.sigmoid, sp.r1, sp.r2, sp.pb, sp.softcap,
                         sp.sink, sp.blocks, sp.keep_first, ext, sp.dist_bias)
    s.copy_(w.view(sp.kv_heads, rep, sp.maps, rep_rows, keys).permute(0, 2, 1, 3, 4).reshape(g, rr, keys))
    return s


def window_attention_products(out, q, k_cache, v_cache, seg: Segments, spec: WindowSpec, min_rows: int):
    """Segments of ``min_rows`` rows or more as banded matrix products: a chunk of rows
    [c0, c1) only sees the keys c0 - window + 1 .. c1 - 1 (or from the start of c0's block;
    plus the kept first positions, gathered in front of the band), so per chunk and key head the
    scores are one product with M = (query heads of the group) x rows, the weights come
    from :func:`band_weights` (fp32) and the sums are a second product with the value
    head.  Operands are fp32 (cached rows are widened), so scores, weights and sums are
    true fp32.  Needs the segments' host copies; writes its rows of ``out``."""
    sp = spec
    start, pos0, kv_len = seg.host
    bs = k_cache.shape[1]
    rep = sp.heads // sp.kv_heads
    gk = sp.kv_heads * sp.maps
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        n = b - a
        if n < min_rows:
            continue
        # without a window a chunk sees every earlier key anyway: long chunks, few launches
        step = PRODUCT_FULL_CHUNK_ROWS if sp.window <= 0 else max(PRODUCT_CHUNK_ROWS, min(sp.window, 1024))
        # the fp32 scores of a chunk ([heads*maps, rows, keys]) stay under PRODUCT_SCORE_BYTES
        span = sp.window if sp.window > 0 else kv_len[s]
        while step > 32 and 4 * sp.heads * sp.maps * step * (step + span) > PRODUCT_SCORE_BYTES:
            step //= 2
        for c0 in range(0, n, step):
            c1 = min(n, c0 + step)
            rows = c1 - c0
            i0 = pos0[s] + c0
            lo = ref.mask_first_key(i0, sp.window, sp.blocks)
            ext = min(sp.keep_first, lo) if sp.window > 0 else 0
            hi = min(kv_len[s], pos0[s] + c1)
            b0, b1 = lo // bs, (hi + bs - 1) // bs
            blocks = seg.block_tables[s, b0:b1].long()
            off = lo - b0 * bs
            k = k_cache.index_select(0, blocks).view((b1 - b0) * bs, gk, sp.dk)[off:off + hi - lo].float()
            v = v_cache.index_select(0, blocks).view((b1 - b0) * bs, sp.kv_heads, sp.dv)[off:off + hi - lo].float()
            if ext:
                # the kept first positions 0 .. ext-1 lie before the band: their rows go in front
                eb = seg.block_tables[s, :(ext + bs - 1) // bs].long()
                k = torch.cat([k_cache.index_select(0, eb).view(-1, gk, sp.dk)[:ext].float(), k], 0)
                v = torch.cat([v_cache.index_select(0, eb).view(-1, sp.kv_heads, sp.dv)[:ext].float(), v], 0)
            # q rows [rows, (g, r, m), dk] -> [(g, m), (r, rows), dk]
            qc = q[a + c0:a + c1].view(rows, sp.kv_heads, rep, sp.maps, sp.dk).permute(1, 3, 2, 0, 4) \
                .reshape(gk, rep * rows, sp.dk)
            sc = torch.bmm(qc, k.permute(1, 2, 0))                       # [gk, rep*rows, keys]
            band_weights(sc, i0, lo, sp, rows, ext)
            # both maps of a group read the same value head: [G, maps*rep*rows, keys] x [G, keys, dv]
            o = torch.bmm(sc.view(sp.kv_heads, sp.maps * rep * rows, ext + hi - lo), v.transpose(0, 1))
            out[a + c0:a + c1] = o.view(sp.kv_heads, sp.maps, rep, rows, sp.dv).permute(3, 0, 2, 1, 4) \
                .reshape(rows, sp.heads * sp.maps, sp.dv)
    return out


# rows of a segment that one pair of banded products covers (at least; a window wider
# than this takes a chunk of its own width, up to 1024 rows)
PRODUCT_CHUNK_ROWS = 256
# rows per chunk when every earlier key is visible (halved until the chunk's scores fit
# PRODUCT_SCORE_BYTES)
PRODUCT_FULL_CHUNK_ROWS = 2048


def diff_combine(a, gate, lam: float, post_scale: float, eps: float, heads: int, dv: int, out_dtype):
    """Two score maps per head -> one output: o = a[:, 2h] - lam * a[:, 2h+1], divided by
    its root mean square over dv, times post_scale * sigmoid(gate[:, h]).  a fp32
    [T, heads*2, dv]; gate [T, heads] (may be a column range); [T, heads*dv]."""
    if a.is_cuda:
        out = torch.empty(a.shape[0], heads * dv, dtype=out_dtype, device=a.device)
        native_mixers().diff_combine(out, a, gate, float(lam), float(post_scale), eps, heads, dv)
        return out
    return ref.diff_combine(a, gate, lam, post_scale, eps, heads, dv, out_dtype)


# ---------------------------------------------------------------------------------
# mixture of experts
# ---------------------------------------------------------------------------------

def moe_topk(z, correction, top: int, groups: int, keep: int):
    """Router: s = softmax(z) (fp32); choice = s + correction; experts outside the
    ``keep`` best of ``groups`` equal groups (by their best choice score) are excluded;
    the ``top`` best choices are returned with their s as weights (not renormalised)."""
    if z.is_cuda:
        t = z.shape[0]
        idx = torch.empty(t, top, dtype=torch.int32, device=z.device)
        wts = torch.empty(t, top, dtype=torch.float32, device=z.device)
        native_mixers().moe_topk(idx, wts, z, correction, top, groups, keep)
        return idx, wts
    return ref.moe_topk(z, correction, top, groups, keep)


def moe_top_logits(z, top: int):
    """Router: the ``top`` largest logits of each fp32 row (ties to the lower index) and,
    as weights, the softmax over just those."""
    if z.is_cuda:
        t = z.shape[0]
        idx = torch.empty(t, top, dtype=torch.int32, device=z.device)
        wts = torch.empty(t, top, dtype=torch.float32, device=z.device)
        native_mixers().moe_top_logits(idx, wts, z, top)
        return idx, wts
    return ref.moe_top_logits(z, top)


def moe_route_top_logits(h, router, bias, top: int):
    """:func:`moe_top_logits` of z = router h + bias (fp32 router [E, width] and bias, h fp32
    or bf16, fp32 accumulation) in one launch: the router of few rows (decode steps)."""
    if h.is_cuda:
        t = h.shape[0]
        idx = torch.empty(t, top, dtype=torch.int32, device=h.device)
        wts = torch.empty(t, top, dtype=torch.float32, device=h.device)
        native_mixers().moe_route_top_logits(idx, wts, h, router, bias, top)
        return idx, wts
    return ref.moe_top_logits(torch.nn.functional.linear(h.float(), router, bias), top)


def moe_pairs(out, h, idx, wts, wgu, wdown, limit: float = 0.0, act: str = "clamp_glu"):
    """Few rows (decode): out (fp32, in place) += sum_k wts[:, k] * expert_{idx[:, k]}(h),
    every (row, expert) pair streaming its expert's first matrix ([gate | up] with the
    clamped GLU, ``act`` "clamp_glu"; or up alone with relu(.)^2, ``act`` "relu_sq") and
    its down matrix; no host round trip, so the step can be captured in a hipGraph."""
    if out.is_cuda:
        native_mixers().moe_pairs(out, h, idx, wts, wgu, wdown, float(limit), act == "relu_sq")
    else:
        ref.moe_pairs(out, h, idx, wts, wgu, wdown, limit, act)


def clamp_swiglu(gu, limit: float):
    """[gate | up (| extra)] rows -> min(gate, limit) * sigmoid(1.702 gate') * (clamp(up) + 1)."""
    if gu.is_cuda:
        ff = gu.shape[1] // 2
        out = torch.empty(gu.shape[0], ff, dtype=gu.dtype, device=gu.device)
        native_mixers().clamp_swiglu(out, gu, float(limit))
        return out
    return ref.clamp_swiglu(gu, limit)


def gelu_glu(gu):
    """[gate | up] rows -> gelu_tanh(gate) * up."""
    if gu.is_cuda:
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
        native_mixers().gelu_glu(out, gu, False)
        return out
    return ref.gelu_glu(gu)


def relu_glu(gu):
    """[gate | up] rows -> relu(gate) * up."""
    if gu.is_cuda:
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
        native_mixers().gelu_glu(out, gu, True)
        return out
    return ref.relu_glu(gu)


def relu_sq(x):
    if x.is_cuda:
        native_mixers().relu_sq(x)
        return x
    return ref.relu_sq(x)


def relu_sq_rows(u, ff: int):
    """relu(u[:, :ff])^2 of wider rows (a column range of a fused product), dense."""
    if u.is_cuda:
        out = torch.empty(u.shape[0], ff, dtype=u.dtype, device=u.device)
        native_mixers().relu_sq_rows(out, u)
        return out
    return ref.relu_sq_rows(u, ff)


def gather_add_rows(out, y, idx, w):
    """out[r] (fp32, in place) += sum_k w[r, k] * y[idx[r, k]]; idx int32 [rows, top]."""
    if out.is_cuda:
        native_mixers().gather_add_rows(out, y, idx, w)
    else:
        ref.gather_add_rows(out, y, idx, w)


def grouped_mm_is_one_product(a, w) -> bool:
    """Whether :func:`grouped_mm` runs as one kernel without reading group sizes on the host."""
    return bool(a.is_cuda and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[1] % 8 == 0)


def grouped_mm(a, w, offsets, counts=None):
    """Rows of ``a`` [M, K] sorted by group; group g's rows (up to ``offsets[g]``, the
    running sum of the group sizes, int32 on the device) times w[g]^T, w [G, N, K] ->
    [M, N] in a's dtype.  bf16 on a GPU with K a multiple of 8 is one grouped MFMA kernel
    (no host round trip); otherwise one vendor product per group (``counts``: the group
    sizes on the host, read from ``offsets`` when not given)."""
    if grouped_mm_is_one_product(a, w):
        out = torch.empty(a.shape[0], w.shape[1], dtype=a.dtype, device=a.device)
        native_mixers().grouped_gemm(out, a.contiguous(), w, offsets)
        return out
    if counts is None:
        ends = offsets.tolist()
        counts = [e - s for s, e in zip([0] + ends[:-1], ends)]
    out = torch.empty(a.shape[0], w.shape[1], dtype=a.dtype, device=a.device)
    s = 0
    for g, n in enumerate(counts):
        if n:
            torch.mm(a[s:s + n], w[g].t(), out=out[s:s + n])
        s += n
    return out


def side_gate(gpre, table, ids, col0: int, sd: int):
    """gelu_tanh(gpre) * table[ids, col0:col0+sd]."""
    if gpre.is_cuda:
        out = torch.empty_like(gpre)
        native_mixers().side_gate(out, gpre, table, ids, col0)
        return out
    return ref.side_gate(gpre, table, ids, col0, sd)


def scale_add_rows(out, y, rows, weights, sigmoid: bool = False):
    """out[rows[i]] += w_i * y[i] (fp32 out; rows None = identity; w = sigmoid(weights)
    if ``sigmoid``).  ``rows`` must not repeat within one call."""
    if out.is_cuda:
        native_mixers().scale_add_rows(out, y, rows, weights, sigmoid)
    else:
        ref.scale_add_rows(out, y, rows, weights, sigmoid)
