"""Reusable sublayers built on :mod:`fasttalk_llm_microservice_amd.ops.mixers`:
latent attention (paged latent cache), windowed attention with sigmoid weights,
windowed differential attention and convolved capped attention with a sink (paged key /
value caches), the channel-decay gated
delta rule and the selective state-space mixer (state slots), dense, gated and
mixture-of-experts feed-forwards and the per-layer token-side input.

Every mixer owns its cache layout: ``alloc_cache(num_blocks, block_size, dtype,
num_slots, device)`` returns what its ``__call__`` takes as ``cache`` (pages indexed by
the engine's block tables, or per-sequence state slots), and ``cache_bytes_per_token``
what a token costs in pages.

Each class takes its sizes and constants as constructor arguments and a ``get(name)``
callable that returns a weight tensor ([out, in] for projections), so a model file only
describes which sublayers it stacks.  Matrix products are vendor GEMMs (``F.linear`` /
``torch.bmm``) in the compute dtype with fp32 accumulation; everything around them runs
in the HIP kernels (GPU) or their PyTorch twins (CPU backend).
"""
from __future__ import annotations

from typing import Callable, List, Optional

import torch
import torch.nn.functional as F

from ..ops import mixers as M

Get = Callable[[str], torch.Tensor]


class StepContext:
    """What a sublayer needs to know about the step: rows' token ids, positions and
    cache slots, and the row segments (one per scheduled sequence)."""

    def __init__(self, ids, positions, slot_mapping, seg: M.Segments):
        self.ids = ids
        self.positions = positions
        self.slot_mapping = slot_mapping
        self.seg = seg


def _state_slots(shapes, num_slots: int, device):
    """(recurrent state, convolution history) fp32, one row per state slot."""
    return tuple(torch.zeros((num_slots,) + tuple(sh), dtype=torch.float32, device=device) for sh in shapes)


class LatentAttention:
    """Multi-head attention whose keys and values are up-projections of one cached
    latent row per token plus one rotated key part shared by all heads.

    The cache holds [rms_norm(latent) | rope(shared key)] per token.  Queries are taken
    into latent space (q_unrotated W_uk, per head), so the attention kernel reads the
    cache rows directly and returns latent-space sums that W_uv maps to the values."""

    def __init__(self, get: Get, width: int, heads: int, dim: int, rot_dim: int, vdim: int,
                 kv_rank: int, scale: float, rot_dims: int, rot_base: float, eps: float,
                 dtype, device, max_pos: int):
        self.heads, self.dn, self.dr, self.dv, self.rank = heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.rot_dims, self.eps, self.dtype = float(scale), int(rot_dims), eps, dtype
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError("rotary dims must be even and within the rotated part")
        self.nq = heads * (dim + rot_dim)
        # q and the latent / shared-key down-projection in one product
        self.wqd = torch.cat([get("q"), get("dkv")], 0).to(device, dtype).contiguous()
        self.dkv_norm = get("dkv.norm").to(device, torch.float32)
        # W_uk [heads, dim, rank] and W_uv^T [heads, rank, vdim], fp32 (small; the
        # absorbed products run on fp32 queries / attention sums)
        self.wuk = get("uk").to(device, torch.float32).view(heads, dim, kv_rank).contiguous()
        self.wuvT = get("uv").to(device, torch.float32).view(heads, vdim, kv_rank) \
            .transpose(1, 2).contiguous()
        self.wo = get("o").to(device, dtype).contiguous()
        self.table = M.rope_table(max_pos, rot_dims, rot_base, device=device)

    # segments of this many rows or more run as matrix products (ops.mixers
    # latent_attention_products), shorter ones and decode rows in the per-row kernel
    PRODUCT_ROWS = 32

    def cache_width(self) -> int:
        return self.rank + self.dr

    def cache_bytes_per_token(self, elem_bytes: int) -> int:
        return self.cache_width() * elem_bytes

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        return torch.zeros(num_blocks, block_size, self.cache_width(), dtype=dtype, device=device)

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        t = h.shape[0]
        qd = F.linear(h, self.wqd)
        q, dkv = qd[:, :self.nq], qd[:, self.nq:]
        M.latent_kv_write(dkv, self.dkv_norm, self.eps, self.table, self.rot_dims, ctx.positions,
                          ctx.slot_mapping, cache, self.rank)
        qn, qr = M.latent_q_rope(q, self.table, self.rot_dims, ctx.positions, self.heads, self.dn,
                                 self.dr)
        qa = torch.bmm(qn.transpose(0, 1), self.wuk)                 # [heads, T, rank]
        seg = ctx.seg
        if seg.host is not None and seg.max_rows >= self.PRODUCT_ROWS:
            # prefill chunks: two tiled products per segment; short segments and decode
            # rows (if any) keep the per-row kernel
            ol = torch.zeros_like(qa)
            M.latent_attention(qa, qr, cache, seg, self.scale, self.rank, skip_from=self.PRODUCT_ROWS,
                               out=ol)
            M.latent_attention_products(ol, qa, qr, cache, seg, self.scale, self.rank,
                                        self.PRODUCT_ROWS, self.dtype)
        else:
            ol = M.latent_attention(qa, qr, cache, seg, self.scale, self.rank)
        o = torch.bmm(ol, self.wuvT)                                  # [heads, T, vdim]
        o = o.transpose(0, 1).reshape(t, self.heads * self.dv).to(self.dtype)
        return F.linear(o, self.wo)


class ChannelDelta:
    """Gated delta rule with a decay per head and key channel, behind short causal
    convolutions on q, k and v; output normed per head and gated."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 taps: int, eps: float, dtype, device):
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kvh, self.dk, self.dv, self.taps = heads, kv_heads, dim, vdim, taps
        self.eps, self.dtype = eps, dtype
        self.wqkv = torch.cat([get("q"), get("k"), get("v")], 0).to(device, dtype).contiguous()
        self.channels = self.wqkv.shape[0]
        self.conv_w = torch.cat([get("q.conv"), get("k.conv"), get("v.conv")], 0) \
            .to(device, torch.float32).contiguous()
        if self.conv_w.shape != (self.channels, taps):
            raise ValueError("convolution weights do not fit the projections")
        a1, g1, b = get("a1"), get("g1"), get("b")
        self.ra, self.rg = a1.shape[0], g1.shape[0]
        # the two low-rank down-projections and beta's projection in one product
        self.wlo = torch.cat([a1, g1, b], 0).to(device, dtype).contiguous()
        self.wa2 = get("a2").to(device, dtype).contiguous()
        self.wg2 = get("g2").to(device, dtype).contiguous()
        self.a_log = get("A_log").to(device, torch.float32)
        self.dt_bias = get("dt_bias").to(device, torch.float32)
        self.norm = get("norm").to(device, torch.float32)
        self.wo = get("o").to(device, dtype).contiguous()

    def state_shapes(self):
        return (self.heads, self.dk, self.dv), (max(self.taps - 1, 0), self.channels)

    def cache_bytes_per_token(self, elem_bytes: int) -> int:
        return 0

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        return _state_slots(self.state_shapes(), num_slots, device)

    def __call__(self, h, ctx: StepContext, state) -> torch.Tensor:
        s_rec, s_conv = state
        qkv = F.linear(h, self.wqkv)
        lo = F.linear(h, self.wlo)
        a = F.linear(lo[:, :self.ra], self.wa2)
        gp = F.linear(lo[:, self.ra:self.ra + self.rg], self.wg2)
        b = lo[:, self.ra + self.rg:].contiguous()
        qkv = M.short_conv_silu(qkv, self.conv_w, s_conv, ctx.seg)
        o = M.gated_delta_rule(qkv, a, b, self.a_log, self.dt_bias, s_rec, ctx.seg, self.heads,
                               self.kvh, self.dk, self.dv)
        y = M.head_rms_gate(o, self.norm, gp, self.eps, self.heads, self.dv, self.dtype)
        return F.linear(y, self.wo)


class WindowedAttention:
    """Grouped-query attention over a sliding window of a paged key cache and a paged
    value cache (common part of :class:`SigmoidAttention` and
    :class:`DifferentialAttention`): the fused q|k|v(|extra) projection, the cache
    layout and the choice between the per-row kernel (decode rows, short segments) and
    banded matrix products (prefill chunks)."""

    # segments of this many rows or more run as banded products
    PRODUCT_ROWS = 32

    def __init__(self, spec: M.WindowSpec, wqkv: torch.Tensor, bias: Optional[torch.Tensor],
                 wo: torch.Tensor, eps: float, dtype, cache_of: Optional[int] = None):
        sp = spec
        if sp.heads % sp.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.spec, self.eps, self.dtype = spec, eps, dtype
        self.nq = sp.heads * sp.maps * sp.dk
        self.nk = sp.kv_heads * sp.maps * sp.dk
        self.nv = sp.kv_heads * sp.dv
        # a layer that reads another layer's keys and values (``cache_of``: that layer's
        # index) projects queries only and owns no pages: the model body hands it the
        # other layer's cache
        self.cache_of = cache_of
        need = self.nq if cache_of is not None else self.nq + self.nk + self.nv
        if wqkv.shape[0] < need or wo.shape[1] != sp.heads * sp.dv:
            raise ValueError("attention projections do not fit the head sizes")
        self.wqkv, self.bias, self.wo = wqkv, bias, wo

    def cache_bytes_per_token(self, elem_bytes: int) -> int:
        return 0 if self.cache_of is not None else (self.nk + self.nv) * elem_bytes

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        if self.cache_of is not None:
            return None
        return (torch.zeros(num_blocks, block_size, self.nk, dtype=dtype, device=device),
                torch.zeros(num_blocks, block_size, self.nv, dtype=dtype, device=device))

    def attend(self, q, ctx: StepContext, cache) -> torch.Tensor:
        """fp32 [T, heads*maps, dv] for fp32 queries [T, heads*maps*dk]."""
        kc, vc = cache
        seg = ctx.seg
        if seg.host is not None and seg.max_rows >= self.PRODUCT_ROWS:
            out = torch.zeros(q.shape[0], self.spec.heads * self.spec.maps, self.spec.dv,
                              dtype=torch.float32, device=q.device)
            if min(b - a for a, b in zip(seg.host[0][:-1], seg.host[0][1:])) < self.PRODUCT_ROWS:
                M.window_attention(q, kc, vc, seg, self.spec, skip_from=self.PRODUCT_ROWS, out=out)
            return M.window_attention_products(out, q, kc, vc, seg, self.spec, self.PRODUCT_ROWS)
        return M.window_attention(q, kc, vc, seg, self.spec)


class SigmoidAttention(WindowedAttention):
    """Windowed attention whose weights are independent sigmoids instead of a softmax:
    w_ij = sigmoid(q_i.k_j * scale - r1_h ln(1 + r2_h (i - j)) + pb_h) for every key in
    the window, and the output is sum_j w_ij v_j as it stands.  q, k and v come from
    biased projections; all rows of q together (and all rows of k together) pass one RMS
    norm with a weight per row; positions enter through the distance term only."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 window: int, scale: float, eps: float, dtype, device):
        f32 = lambda n: get(n).to(device, torch.float32).contiguous()   # noqa: E731
        spec = M.WindowSpec(heads, kv_heads, dim, vdim, int(window), float(scale), maps=1, sigmoid=True,
                            r1=f32("r1"), r2=f32("r2"), pb=f32("pb"))
        wqkv = torch.cat([get("q"), get("k"), get("v")], 0).to(device, dtype).contiguous()
        bias = torch.cat([get("q.b"), get("k.b"), get("v.b")], 0).to(device, dtype).contiguous()
        super().__init__(spec, wqkv, bias, get("o").to(device, dtype).contiguous(), eps, dtype)
        self.q_norm, self.k_norm = f32("q.norm"), f32("k.norm")
        if self.q_norm.numel() != self.nq or self.k_norm.numel() != self.nk or spec.r1.numel() != heads:
            raise ValueError("attention norm / bias tensors do not fit the head sizes")

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        qkv = F.linear(h, self.wqkv, self.bias)
        q = M.attn_prep(qkv, self.nq, self.nk, self.q_norm, self.k_norm, self.eps, None, 0, self.spec.dk,
                        ctx.positions, ctx.slot_mapping, cache[0], cache[1])
        o = self.attend(q, ctx, cache)
        return F.linear(o.view(h.shape[0], -1).to(self.dtype), self.wo)


class DifferentialAttention(WindowedAttention):
    """Windowed attention that subtracts a second softmax map from the first.  For each
    head in turn, q and k hold the rows of its map-0 projection and then of its map-1
    projection; both maps weight one shared set of values, giving a_0 and a_1.  Output
    per head: o = a_0 - lam a_1 with the layer constant
    lam = exp(<lq1, lk1>) - exp(<lq2, lk2>) + diff; then o / rms(o) * (1 - diff) *
    sigmoid(g_h), where g = W_g x is one gate logit per head taken from the mixer's input.
    The first ``rot_dims`` entries of every map's q and k rows are rotated by position
    (frequencies optionally rescaled by wavelength, :func:`ops.mixers_ref.scale_frequencies`)."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 window: int, scale: float, diff: float, rot_dims: int, rot_base: float, rot_scaling,
                 eps: float, dtype, device, max_pos: int):
        spec = M.WindowSpec(heads, kv_heads, dim, vdim, int(window), float(scale), maps=2)
        # the gate's rows ride on the fused projection
        wqkv = torch.cat([get("q"), get("k"), get("v"), get("g")], 0).to(device, dtype).contiguous()
        super().__init__(spec, wqkv, None, get("o").to(device, dtype).contiguous(), eps, dtype)
        if rot_dims % 2 or rot_dims > dim or wqkv.shape[0] != self.nq + self.nk + self.nv + heads:
            raise ValueError("differential attention sizes do not fit")
        f = lambda n: get(n).to(torch.float32).cpu()   # noqa: E731
        self.diff = float(diff)
        self.lam = float(torch.exp((f("lq1") * f("lk1")).sum()) - torch.exp((f("lq2") * f("lk2")).sum())
                         + torch.tensor(self.diff, dtype=torch.float32))
        self.rot_dims = int(rot_dims)
        self.table = M.rope_table(max_pos, rot_dims, rot_base, device=device, scaling=rot_scaling) \
            if rot_dims else None

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        qkvg = F.linear(h, self.wqkv)
        n = self.nq + self.nk + self.nv
        q = M.attn_prep(qkvg[:, :n], self.nq, self.nk, None, None, self.eps, self.table, self.rot_dims,
                        self.spec.dk, ctx.positions, ctx.slot_mapping, cache[0], cache[1])
        a = self.attend(q, ctx, cache)
        o = M.diff_combine(a, qkvg[:, n:], self.lam, 1.0 - self.diff, self.eps, self.spec.heads,
                           self.spec.dv, self.dtype)
        return F.linear(o, self.wo)


class ConvSinkAttention(WindowedAttention):
    """Grouped-query softmax attention over every earlier key (or a window of them) whose
    q, k and v each pass a short per-channel causal convolution over time right after
    their projection (no bias, no activation; the last taps-1 projected rows of a sequence
    live in its state slot).  Each head's q and k are divided by their root mean square
    and multiplied by one weight vector shared by all heads.  Positions do not enter the
    scores: s = softcap tanh(q.k scale / softcap), and the softmax's denominator carries
    one extra unit, exp(sink) with sink = 0 -- a key that is always visible and has no
    value, so a row's weights may sum to less than one."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int,
                 scale: float, softcap: float, eps: float, dtype, device, window: int = 0,
                 sink: Optional[float] = 0.0):
        f32 = lambda n: get(n).to(device, torch.float32).contiguous()   # noqa: E731
        spec = M.WindowSpec(heads, kv_heads, dim, vdim, int(window), float(scale), maps=1,
                            softcap=float(softcap or 0.0), sink=sink)
        wqkv = torch.cat([get("q"), get("k"), get("v")], 0).to(device, dtype).contiguous()
        super().__init__(spec, wqkv, None, get("o").to(device, dtype).contiguous(), eps, dtype)
        self.taps = int(taps)
        self.conv_w = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")], 0).contiguous()
        self.q_norm, self.k_norm = f32("q.norm"), f32("k.norm")
        self.channels = self.nq + self.nk + self.nv
        if wqkv.shape != (self.channels, width) or self.conv_w.shape != (self.channels, self.taps) \
                or self.q_norm.numel() != dim or self.k_norm.numel() != dim:
            raise ValueError("attention projections, convolutions or norms do not fit the head sizes")

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        """(paged keys, paged values, projected-row history per state slot)."""
        return super().alloc_cache(num_blocks, block_size, dtype, num_slots, device) + \
            _state_slots(((max(self.taps - 1, 0), self.channels),), num_slots, device)

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        kc, vc, hist = cache
        qkv = F.linear(h, self.wqkv)
        q = M.conv_attn_prep(qkv, self.nq, self.nk, self.conv_w, hist, ctx.seg, self.q_norm, self.k_norm,
                             self.eps, self.spec.dk, ctx.slot_mapping, kc, vc)
        o = self.attend(q, ctx, (kc, vc))
        return F.linear(o.view(h.shape[0], -1).to(self.dtype), self.wo)


class BiasedWindowAttention(WindowedAttention):
    """Grouped-query softmax attention without rotation.  All rows of q together (and all
    rows of k together) pass one RMS norm with a weight per row; the score of query i and
    key j gains rel[bucket(i - j), head] from a table of ``rel.shape[0]`` rows -- distances
    below half the rows have a row each, larger ones share rows in logarithmic steps up to
    ``bias_reach`` (:func:`ops.mixers.distance_bias_table`); a position sees the last
    ``window`` positions and, whatever the window, the first ``keep_first`` of the
    sequence.  The concatenated heads are multiplied by sigmoid(W_g h) before the output
    projection.  With ``cache_of`` the layer has no k / v projections of its own and
    attends to the pages of the layer it names (keys as cached there, after that layer's
    norm)."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                 keep_first: int, scale: float, bias_reach: int, eps: float, dtype, device,
                 cache_of: Optional[int] = None):
        f32 = lambda n: get(n).to(device, torch.float32).contiguous()   # noqa: E731
        rel = f32("rel")
        if rel.dim() != 2 or rel.shape[1] != heads:
            raise ValueError("distance bias table does not fit the heads")
        spec = M.WindowSpec(heads, kv_heads, dim, vdim, int(window), float(scale), maps=1,
                            keep_first=int(keep_first), dist_bias=M.distance_bias_table(rel, int(bias_reach)))
        parts = [get("q")] + ([] if cache_of is not None else [get("k"), get("v")]) + [get("g")]
        wqkv = torch.cat(parts, 0).to(device, dtype).contiguous()
        super().__init__(spec, wqkv, None, get("o").to(device, dtype).contiguous(), eps, dtype, cache_of)
        self.q_norm = f32("q.norm")
        self.k_norm = None if cache_of is not None else f32("k.norm")
        self.ng = heads * vdim
        own = 0 if cache_of is not None else self.nk + self.nv
        if wqkv.shape != (self.nq + own + self.ng, width) or self.q_norm.numel() != self.nq or \
                (self.k_norm is not None and self.k_norm.numel() != self.nk):
            raise ValueError("attention projections or norms do not fit the head sizes")
        self.n_in = self.nq + own

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        p = F.linear(h, self.wqkv)
        if self.cache_of is not None:
            q = M.attn_prep(p[:, :self.nq], self.nq, 0, self.q_norm, None, self.eps, None, 0, self.spec.dk,
                            ctx.positions, ctx.slot_mapping, None, None)
        else:
            q = M.attn_prep(p[:, :self.n_in], self.nq, self.nk, self.q_norm, self.k_norm, self.eps, None, 0,
                            self.spec.dk, ctx.positions, ctx.slot_mapping, cache[0], cache[1])
        o = self.attend(q, ctx, cache)
        return F.linear(M.sigmoid_gate(o.view(h.shape[0], -1), p[:, self.n_in:], self.dtype), self.wo)


class RotaryBlockAttention(WindowedAttention):
    """Grouped-query softmax attention with rotary positions on the first ``rot_dims``
    entries of every head (entry i paired with i + rot_dims/2; frequencies optionally
    ramped down for long contexts, ``rot_ramp`` = (factor, original, fast, slow) of
    :func:`ops.mixers.ramp_frequencies`).  The sequence is cut into blocks of ``window``
    positions counted from position 0, and a position sees the earlier positions of its
    own block only (``window`` 0: every earlier position)."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                 scale: float, rot_dims: int, rot_base: float, rot_ramp, eps: float, dtype, device, max_pos: int):
        spec = M.WindowSpec(heads, kv_heads, dim, vdim, int(window), float(scale), maps=1, blocks=True)
        wqkv = torch.cat([get("q"), get("k"), get("v")], 0).to(device, dtype).contiguous()
        super().__init__(spec, wqkv, None, get("o").to(device, dtype).contiguous(), eps, dtype)
        if rot_dims % 2 or rot_dims > dim or wqkv.shape != (self.nq + self.nk + self.nv, width):
            raise ValueError("attention sizes do not fit")
        self.rot_dims = int(rot_dims)
        self.table = M.rope_table(max_pos, rot_dims, rot_base, device=device, ramp=rot_ramp) if rot_dims else None

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        qkv = F.linear(h, self.wqkv)
        q = M.attn_prep(qkv, self.nq, self.nk, None, None, self.eps, self.table, self.rot_dims, self.spec.dk,
                        ctx.positions, ctx.slot_mapping, cache[0], cache[1])
        o = self.attend(q, ctx, cache)
        return F.linear(o.view(h.shape[0], -1).to(self.dtype), self.wo)


class GatedLinearAttention:
    """Linear attention with a decay per head and key channel: S <- diag(alpha) S + k v^T,
    o = S^T q with q = W_q h dk^-1/2, alpha = sigmoid(W_a2 W_a1 h + b)^(1/tau).  Each head's
    o is divided by its root mean square and multiplied by one weight vector shared by the
    heads, the concatenated heads by silu(W_g h), then the output projection.  The state
    [heads, dk, dv] is fp32 and lives in the sequence's state slot."""

    def __init__(self, get: Get, width: int, heads: int, dim: int, vdim: int, tau: float, eps: float,
                 dtype, device):
        self.heads, self.dk, self.dv, self.tau, self.eps, self.dtype = heads, dim, vdim, float(tau), eps, dtype
        a1 = get("a1")
        self.nqkv = heads * (2 * dim + vdim)
        self.ng = heads * vdim
        # q | k | v | output gate | the decay's low-rank down-projection in one product
        self.win = torch.cat([get("q"), get("k"), get("v"), get("g"), a1], 0).to(device, dtype).contiguous()
        self.wa2 = get("a2").to(device, dtype).contiguous()
        self.a_bias = get("a2.b").to(device, torch.float32).contiguous()
        self.norm = get("norm").to(device, torch.float32).contiguous()
        self.wo = get("o").to(device, dtype).contiguous()
        if self.win.shape != (self.nqkv + self.ng + a1.shape[0], width) or \
                self.wa2.shape != (heads * dim, a1.shape[0]) or self.a_bias.numel() != heads * dim or \
                self.norm.numel() != vdim or self.wo.shape[1] != self.ng:
            raise ValueError("linear-attention projections do not fit the head sizes")

    def cache_bytes_per_token(self, elem_bytes: int) -> int:
        return 0

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        return _state_slots(((self.heads, self.dk, self.dv),), num_slots, device)[0]

    def __call__(self, h, ctx: StepContext, state) -> torch.Tensor:
        p = F.linear(h, self.win)
        a = F.linear(p[:, self.nqkv + self.ng:], self.wa2)
        o = M.gated_linear_attention(p, a, self.a_bias, self.tau, state, ctx.seg, self.heads, self.dk, self.dv)
        y = M.head_rms_gate(o, self.norm, p[:, self.nqkv:self.nqkv + self.ng], self.eps, self.heads, self.dv,
                            self.dtype, silu=True)
        return F.linear(y, self.wo)


class SideBySide:
    """Two mixers that read the same input; each output is divided by its root mean
    square over the model width and multiplied by a weight vector of its own, and the
    result is ``scale`` (one half) times their sum, in fp32.  The cache is the pair of the
    two mixers' caches."""

    def __init__(self, left, right, w_left: torch.Tensor, w_right: torch.Tensor, eps: float, device,
                 scale: float = 0.5):
        self.left, self.right, self.eps, self.scale = left, right, eps, float(scale)
        self.w_left = w_left.to(device, torch.float32).contiguous()
        self.w_right = w_right.to(device, torch.float32).contiguous()

    def cache_bytes_per_token(self, elem_bytes: int) -> int:
        return self.left.cache_bytes_per_token(elem_bytes) + self.right.cache_bytes_per_token(elem_bytes)

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        return (self.left.alloc_cache(num_blocks, block_size, dtype, num_slots, device),
                self.right.alloc_cache(num_blocks, block_size, dtype, num_slots, device))

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        a = self.left(h, ctx, cache[0])
        b = self.right(h, ctx, cache[1])
        return M.dual_rms_mean(a, b, self.w_left, self.w_right, self.eps, self.scale)


class StateSpaceMixer:
    """Selective state-space mixer with a scalar decay per head (state-space duality
    form): one input projection [z | x | B | C | dt], a short causal convolution with
    bias and SiLU over x|B|C, the recurrence S <- exp(-exp(A) dt) S + dt B x^T,
    y = S^T C + D x with dt = softplus(dt + dt_bias), then y silu(z), an RMS norm in
    ``norm_groups`` equal parts with a weight, and the output projection."""

    def __init__(self, get: Get, width: int, heads: int, vdim: int, state: int, groups: int, taps: int,
                 norm_groups: int, eps: float, dtype, device):
        self.heads, self.dv, self.n, self.groups, self.taps = heads, vdim, state, groups, taps
        self.norm_groups, self.eps, self.dtype = norm_groups, eps, dtype
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        if heads % groups or self.inner % norm_groups:
            raise ValueError("state-space heads / groups do not divide")
        f32 = lambda n: get(n).to(device, torch.float32).contiguous()   # noqa: E731
        self.win = get("in").to(device, dtype).contiguous()
        if self.win.shape[0] != self.inner + self.channels + heads:
            raise ValueError("state-space input projection does not fit its sizes")
        self.conv_w, self.conv_b = f32("conv"), f32("conv.b")
        if self.conv_w.shape != (self.channels, taps):
            raise ValueError("convolution weights do not fit the projection")
        self.a_log, self.dt_bias, self.d_skip, self.norm = f32("A_log"), f32("dt_bias"), f32("D"), f32("norm")
        self.wo = get("o").to(device, dtype).contiguous()

    def state_shapes(self):
        return (self.heads, self.n, self.dv), (max(self.taps - 1, 0), self.channels)

    def cache_bytes_per_token(self, elem_bytes: int) -> int:
        return 0

    def alloc_cache(self, num_blocks, block_size, dtype, num_slots, device):
        return _state_slots(self.state_shapes(), num_slots, device)

    def __call__(self, h, ctx: StepContext, state) -> torch.Tensor:
        s_rec, s_conv = state
        p = F.linear(h, self.win)
        z = p[:, :self.inner]
        xbc = M.short_conv_silu(p[:, self.inner:self.inner + self.channels], self.conv_w, s_conv, ctx.seg,
                                bias=self.conv_b)
        y = M.ssd_scan(xbc, p[:, self.inner + self.channels:], self.a_log, self.dt_bias, self.d_skip, s_rec,
                       ctx.seg, self.heads, self.groups, self.n, self.dv)
        y = M.gate_group_norm(y, z, self.norm, self.eps, self.norm_groups, self.dtype)
        return F.linear(y, self.wo)


class GatedFF:
    """down(act(gate h) * (up h)), act = gelu_tanh or relu."""

    def __init__(self, get: Get, dtype, device, act: str = "gelu_tanh"):
        if act not in ("gelu_tanh", "relu"):
            raise ValueError("unknown feed-forward activation")
        self.wgu, self.down = _glu_weights(get, "", dtype, device)
        self.glu = M.gelu_glu if act == "gelu_tanh" else M.relu_glu

    def __call__(self, h, ctx=None) -> torch.Tensor:
        return F.linear(self.glu(F.linear(h, self.wgu)), self.down)


class DenseFF:
    """down(relu(up h)^2)."""

    def __init__(self, get: Get, dtype, device):
        self.up = get("up").to(device, dtype).contiguous()
        self.down = get("down").to(device, dtype).contiguous()

    def __call__(self, h, ctx=None) -> torch.Tensor:
        return F.linear(M.relu_sq(F.linear(h, self.up)), self.down)


def _glu_weights(get: Get, prefix: str, dtype, device, extra: Optional[torch.Tensor] = None):
    parts = [get(prefix + "gate"), get(prefix + "up")] + ([extra] if extra is not None else [])
    return (torch.cat(parts, 0).to(device, dtype).contiguous(),
            get(prefix + "down").to(device, dtype).contiguous())


class MoEFF:
    """Top-k mixture of small feed-forward experts with an optional shared expert that
    runs for every token and is scaled by sigmoid(w_sg . h), one number per token.

    Two designs of routing and expert are served (``routing`` / ``act``):

    * ``"grouped_softmax"`` + ``"clamp_glu"``: softmax over all experts, an additive
      selection bias (``correction``) that does not enter the weights, only the ``keep``
      best of ``groups`` groups eligible; expert g = min(W_gate h, limit),
      u = clamp(W_up h, +-limit), y = g sigmoid(1.702 g) (u + 1), out = W_down y;
    * ``"top_logits"`` + ``"relu_sq"``: logits z = W_router h + b; the ``top`` largest are
      chosen and weighted by the softmax over just those; expert out =
      W_down relu(W_up h)^2.

    Router logits are fp32 in both."""

    def __init__(self, get: Get, experts: int, top: int, limit: float, groups: int, keep: int,
                 shared_limit: Optional[float], dtype, device, routing: str = "grouped_softmax",
                 act: str = "clamp_glu", shared: Optional[bool] = None):
        if groups < 1 or experts % groups or not 1 <= keep <= groups or top > experts // groups * keep:
            raise ValueError("expert groups do not fit the expert count")
        if routing not in ("grouped_softmax", "top_logits") or act not in ("clamp_glu", "relu_sq"):
            raise ValueError("unknown routing or expert activation")
        self.e, self.top, self.limit, self.groups, self.keep = experts, top, float(limit), groups, keep
        self.dtype, self.routing, self.act = dtype, routing, act
        self.router = get("router").to(device, torch.float32).contiguous()
        if routing == "grouped_softmax":
            self.correction = get("correction").to(device, torch.float32).contiguous()
            self.router_bias = None
        else:
            self.router_bias = get("router.b").to(device, torch.float32).contiguous()
        if act == "clamp_glu":
            firsts, downs = zip(*[_glu_weights(get, f"e{i}.", dtype, device) for i in range(experts)])
        else:
            firsts = [get(f"e{i}.up").to(device, dtype) for i in range(experts)]
            downs = [get(f"e{i}.down").to(device, dtype) for i in range(experts)]
        self.wgu = torch.stack(list(firsts)).contiguous()      # [E, 2 ff | ff, width]
        self.wdown = torch.stack(list(downs)).contiguous()    # [E, width, ff]
        self.shared = None
        if shared is None:
            shared = shared_limit is not None
        if shared:
            # the shared expert's per-token gate logit rides as one more output row
            if act == "clamp_glu":
                self.shared = _glu_weights(get, "shared.", dtype, device, extra=get("shared.sg"))
            else:
                self.shared = (torch.cat([get("shared.up"), get("shared.sg")], 0).to(device, dtype).contiguous(),
                               get("shared.down").to(device, dtype).contiguous())
            self.shared_limit = float(shared_limit or 0.0)

    def route(self, h):
        if self.routing == "grouped_softmax":
            z = F.linear(h.float(), self.router)
            return M.moe_topk(z, self.correction, self.top, self.groups, self.keep)
        if h.shape[0] <= self.PAIR_ROWS:
            return M.moe_route_top_logits(h, self.router, self.router_bias, self.top)
        return M.moe_top_logits(F.linear(h.float(), self.router, self.router_bias), self.top)

    def _act(self, u):
        return M.clamp_swiglu(u, self.limit) if self.act == "clamp_glu" else M.relu_sq(u)

    def __call__(self, h, ctx=None) -> torch.Tensor:
        t, width = h.shape
        out = torch.zeros(t, width, dtype=torch.float32, device=h.device)
        idx, wts = self.route(h)
        if t <= self.PAIR_ROWS:
            # decode-size steps: per-pair weight streaming, nothing read back on the host
            M.moe_pairs(out, h, idx, wts, self.wgu, self.wdown, self.limit, self.act)
            return self._shared(out, h)
        # rows sorted by expert: each expert's rows are one group of two grouped products
        flat = idx.view(-1).long()
        order = torch.argsort(flat, stable=True)
        offs = torch.bincount(flat, minlength=self.e).cumsum(0).int()
        hs = h.index_select(0, order // self.top)
        # group sizes on the host only where a product runs group by group
        counts = None if M.grouped_mm_is_one_product(hs, self.wgu) and self.wdown.shape[2] % 8 == 0 \
            else torch.bincount(flat, minlength=self.e).tolist()   # K of both products a multiple of 8
        y = self._act(M.grouped_mm(hs, self.wgu, offs, counts))
        d = M.grouped_mm(y, self.wdown, offs, counts)
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        M.gather_add_rows(out, d, inv.view(t, self.top).int(), wts)
        return self._shared(out, h)

    # rows up to which every (row, expert) pair streams its expert's weights (decode);
    # above, rows are sorted by expert and run as grouped products
    PAIR_ROWS = 64

    def _shared(self, out, h):
        if self.shared is not None:
            w1, wdown = self.shared
            u = F.linear(h, w1)
            if self.act == "clamp_glu":
                y = M.clamp_swiglu(u, self.shared_limit)
            else:
                y = M.relu_sq_rows(u, u.shape[1] - 1)
            M.scale_add_rows(out, F.linear(y, wdown), None, u[:, -1].contiguous(), sigmoid=True)
        return out


class TokenSide:
    """Per-layer token input: y = proj(gelu_tanh(gate x) * side_embed[token, part]);
    the caller adds rms_norm(y) * norm to the residual."""

    def __init__(self, get: Get, table: torch.Tensor, col0: int, dim: int, dtype, device):
        self.table, self.col0, self.dim = table, col0, dim
        self.gate = get("gate").to(device, dtype).contiguous()
        self.proj = get("proj").to(device, dtype).contiguous()
        self.norm = get("norm").to(device, torch.float32)

    def __call__(self, xc, ctx: StepContext) -> torch.Tensor:
        g = M.side_gate(F.linear(xc, self.gate), self.table, ctx.ids, self.col0, self.dim)
        return F.linear(g, self.proj)
