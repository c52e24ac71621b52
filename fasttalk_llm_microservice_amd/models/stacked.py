"""The common body of the models that stack sublayers from :mod:`.mixers` on an fp32
residual stream: layer *runs* (a layer may run more than once, or borrow another
layer's weights, and every run owns its cache or state), pre- and post-norms around
each sublayer fused into one kernel between sublayers, paged caches and state slots
allocated by the mixers themselves, final norm and the vocabulary product.

A subclass parses its configuration, says which layers run in which order
(``cfg.runs()``: (layer index, row of ``loop.step`` added right before it or None)) and
builds the layer list in ``load_tensors``.

Per run, with x the residual:  x += norm1b(mixer(norm1 x));
x += norm2b(ff(norm2 x)) (if the layer has a feed-forward);
x += rms(side(x, token)) * side.norm (if it has a token-side input).

A model with ``norm_style = "layer_post"`` has no norm in front of its sublayers: they
read x itself, and a layer norm with weight and bias sits on each sublayer's output,
x += ln1(mixer(x)); x += ln2(ff(x)); the embedding rows (plus, optionally, a sinusoidal
position vector) pass a layer norm before the first layer, and the final norm is a layer
norm too.

A model with ``norm_style = "shared_pre"`` has one RMS norm per layer that both sublayers
read, and their outputs are added together: h = norm1(x); x += residual_mult *
(mixer(h) + ff(h)).  The add and the next layer's norm are one kernel.

Embedding extras: a pair table (``pair_embed``: a row chosen by a hash of the previous and
the current token is added to the embedding row; the previous token of a sequence is kept
in its state slot) and a scale on the logits; a model without a ``head`` tensor uses its
embedding table as the head.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional

import torch
import torch.nn.functional as F

from ..ops import mixers as M
from ..parallel.comm import SINGLE, TPComm
from . import weights as W
from .mixers import StepContext


@dataclasses.dataclass
class StackedLayer:
    kind: str
    norm1: torch.Tensor
    norm1b: torch.Tensor
    mixer: object
    norm2: Optional[torch.Tensor] = None
    norm2b: Optional[torch.Tensor] = None
    ff: Optional[object] = None
    side: Optional[object] = None
    # biases of the output norms (layer-norm models)
    bias1: Optional[torch.Tensor] = None
    bias2: Optional[torch.Tensor] = None


class StackedCache:
    """Per layer run, what its mixer's ``alloc_cache`` returned: paged tensors
    [num_blocks, block_size, ...] and / or per-slot state tensors [slots, ...]."""

    def __init__(self, per_run: list, extra: Optional[dict] = None):
        self.per_run = per_run
        self.extra = extra or {}      # state that belongs to no layer (per-slot tensors)

    def tensors(self):
        seen = set()

        def walk(c):
            if isinstance(c, torch.Tensor):
                if id(c) not in seen:      # a run that reads another run's pages holds the same tensors
                    seen.add(id(c))
                    yield c
            elif c is not None:
                for e in c:
                    yield from walk(e)

        yield from walk(self.per_run)
        yield from walk(list(self.extra.values()))


class StackedModel:
    needs_state_slots = True     # the runner hands every sequence a state slot
    supports_graphs = True
    family = "stacked"
    norm_style = "rms_pre_post"   # or "layer_post"

    def __init__(self, cfg, device, dtype=torch.bfloat16, comm: TPComm = SINGLE,
                 max_model_len: int = 8192, quantization: Optional[str] = None):
        if comm.world_size != 1:
            raise ValueError(f"{self.family} runs on one device (tensor parallelism is not implemented)")
        if quantization:
            raise ValueError(f"{self.family} has no quantized weight path")
        self.cfg, self.device, self.dtype, self.comm = cfg, torch.device(device), dtype, comm
        self.tp, self.rank = 1, 0
        self.max_model_len = max_model_len
        self.runs = cfg.runs()
        self.layers: List[StackedLayer] = []
        self.embed = self.head = self.final_norm = self.loop_step = None
        self.embed_scale = 1.0
        self.pos_freqs = None                   # fp32 sinusoid frequencies (position vector added to the embedding)
        self.embed_norm = None                  # (weight, bias) of the layer norm after the embedding
        self.final_bias = None
        self.logit_softcap = 0.0
        self.logit_scale = 1.0
        self.residual_mult = 1.0                # shared_pre: x += residual_mult * (mixer + ff)
        self.pair_embed = None                  # (table, mul_prev, mul_cur, buckets)
        self.vocab_pad = 0
        self.mark_at = None
        self.layer_tap: Optional[list] = None   # tests: fp32 residual after every layer run
        self.invariant = False
        self._mm_out_dtype = True
        if self.device.type == "cuda":
            # true fp32 / fp32-accumulated products from the vendor library
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = False

    # ------------------------------------------------------------------ weights
    def load_tensors(self, get, has=lambda n: True):
        raise NotImplementedError

    def random_tensors(self, seed: int, device):
        raise NotImplementedError

    def load_head(self, get, has=lambda n: True):
        """embed and head (rows padded to a multiple of 8) from the checkpoint; without a
        ``head`` tensor the embedding table is the head."""
        dev, dt = self.device, self.dtype
        self.embed = get("embed").to(dev, dt).contiguous()
        head = (get("head") if has("head") else get("embed")).to(dev, dt)
        # the sampler reads logits rows in groups of 8: zero rows pad the head, and their
        # logits are set to -inf (never sampled; callers that want logits cut them off)
        self.vocab_pad = (-head.shape[0]) % 8
        if self.vocab_pad:
            head = torch.cat([head, torch.zeros(self.vocab_pad, head.shape[1], dtype=dt, device=dev)], 0)
        elif not has("head"):
            head = self.embed                    # one table for both
        self.head = head.contiguous()

    def norm_weight(self, t: torch.Tensor) -> torch.Tensor:
        """fp32 [width] weight of a residual-stream norm; a checkpoint that stores one
        number per norm has it repeated over the width."""
        t = t.to(self.device, torch.float32)
        if t.numel() == 1:
            t = t.reshape(1).expand(self.cfg.hidden_size)
        return t.contiguous()

    def load_checkpoint(self, ckpt_dir: str):
        idx = W.SafetensorsIndex(ckpt_dir)
        return self.load_tensors(idx.get, idx.has)

    def init_random(self, seed: int = 0, **_):
        on = self.device if self.device.type == "cuda" else "cpu"
        t = self.random_tensors(seed, on)
        return self.load_tensors(t.__getitem__, t.__contains__)

    def resident_weight_bytes(self) -> int:
        seen, total = set(), 0
        stack = [self.__dict__]
        while stack:
            o = stack.pop()
            vals = o.values() if isinstance(o, dict) else o if isinstance(o, (list, tuple)) else \
                vars(o).values() if hasattr(o, "__dict__") else ()
            for v in vals:
                if isinstance(v, torch.Tensor):
                    if v.data_ptr() not in seen:
                        seen.add(v.data_ptr())
                        total += v.numel() * v.element_size()
                elif isinstance(v, (dict, list, tuple)) or hasattr(v, "__dict__") and \
                        type(v).__module__.startswith(__package__):
                    stack.append(v)
        return total


    # ------------------------------------------------------------------ cache / state
    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(self.layers[i].mixer.cache_bytes_per_token(dtype_bytes) for i, _ in self.runs)

    def kv_block_bytes(self, block_size: int, dtype) -> int:
        es = torch.tensor([], dtype=dtype).element_size()
        return max(1, self.kv_bytes_per_token(es) * block_size)

    def allocate_kv_cache(self, num_blocks: int, block_size: int, dtype=None, num_slots: int = 1):
        """One cache / state per layer RUN (a layer that runs twice owns two)."""
        dt = dtype or self.dtype
        if dt not in (torch.float32, torch.bfloat16):
            raise ValueError("paged caches are kept in the compute dtype")
        per_run = [self.layers[i].mixer.alloc_cache(num_blocks, block_size, dt, num_slots, self.device)
                   for i, _ in self.runs]
        # a mixer that reads another layer's keys and values gets that layer's (first) run's pages
        for r, (i, _) in enumerate(self.runs):
            src = getattr(self.layers[i].mixer, "cache_of", None)
            if src is not None:
                owner = next(q for q, (j, _) in enumerate(self.runs) if j == src)
                per_run[r] = per_run[owner]
        extra = {}
        if self.pair_embed is not None:
            extra["last_token"] = torch.full((max(num_slots, 1),), -1, dtype=torch.int32, device=self.device)
        return StackedCache(per_run, extra)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, meta, caches: StackedCache) -> torch.Tensor:
        """Final-normed hidden rows (compute dtype) at ``meta.logits_indices``."""
        cfg, dt, eps = self.cfg, self.dtype, self.cfg.rms_norm_eps
        seg = meta.segments
        if seg is None:
            raise ValueError("this model needs the step's row segments (AttnMeta.segments)")
        ctx = StepContext(input_ids, meta.positions, meta.slot_mapping, seg)
        if self.norm_style == "layer_post":
            return self._forward_layer_post(input_ids, meta, ctx, caches)
        if self.norm_style == "shared_pre":
            return self._forward_shared_pre(input_ids, meta, ctx, caches)
        x = M.embed_rows(input_ids, self.embed, self.embed_scale)
        tap = self.layer_tap
        fuse_step = tap is None
        h = None
        nruns = len(self.runs)
        mark = self.mark_at
        for r, (li, step) in enumerate(self.runs):
            if mark is not None and r == mark[0]:
                mark[1].record()
            L = self.layers[li]
            if h is None:   # first run, or the step vector was not fused into the last kernel
                vec = self.loop_step[step] if step is not None and (r == 0 or not fuse_step) else None
                h = M.rms_norm_rows(x, L.norm1, eps, dt, add_vec=vec)
            y = L.mixer(h, ctx, caches.per_run[r])
            nxt = self.runs[r + 1] if r + 1 < nruns else None
            nvec = self.loop_step[nxt[1]] if nxt is not None and nxt[1] is not None and fuse_step else None
            nw = self.layers[nxt[0]].norm1 if nxt is not None and (fuse_step or nxt[1] is None) else None
            last = L.ff is None and L.side is None
            h, xc = M.add_rms_norm_rows(x, y, L.norm1b, eps,
                                        add_vec=nvec if last else None,
                                        next_w=L.norm2 if L.ff is not None else (nw if last else None),
                                        out_dtype=dt, want_cast=L.ff is None and L.side is not None)
            if L.ff is not None:
                y = L.ff(h, ctx)
                last = L.side is None
                h, xc = M.add_rms_norm_rows(x, y, L.norm2b, eps, add_vec=nvec if last else None,
                                            next_w=nw if last else None, out_dtype=dt,
                                            want_cast=L.side is not None)
            if L.side is not None:
                y = L.side(xc, ctx)
                h, _ = M.add_rms_norm_rows(x, y, L.side.norm, eps, add_vec=nvec, next_w=nw,
                                           out_dtype=dt)
            if tap is not None:
                tap.append(x.clone())
        idx = meta.logits_indices
        rows = x.index_select(0, idx) if idx.numel() != x.shape[0] else x
        if rows.shape[0] == 0:
            return rows.to(dt)
        return M.rms_norm_rows(rows, self.final_norm, eps, dt)

    def _forward_layer_post(self, input_ids, meta, ctx, caches: StackedCache) -> torch.Tensor:
        dt, eps = self.dtype, self.cfg.rms_norm_eps
        x = M.embed_rows(input_ids, self.embed, self.embed_scale, meta.positions, self.pos_freqs)
        h = M.add_layer_norm_rows(x, None, self.embed_norm[0], self.embed_norm[1], eps, dt) \
            if self.embed_norm is not None else (x if dt == torch.float32 else x.to(dt))
        tap, mark = self.layer_tap, self.mark_at
        for r, (li, _) in enumerate(self.runs):
            if mark is not None and r == mark[0]:
                mark[1].record()
            L = self.layers[li]
            h = M.add_layer_norm_rows(x, L.mixer(h, ctx, caches.per_run[r]), L.norm1b, L.bias1, eps, dt)
            if L.ff is not None:
                h = M.add_layer_norm_rows(x, L.ff(h, ctx), L.norm2b, L.bias2, eps, dt)
            if tap is not None:
                tap.append(x.clone())
        idx = meta.logits_indices
        rows = x.index_select(0, idx) if idx.numel() != x.shape[0] else x
        if rows.shape[0] == 0:
            return rows.to(dt)
        return M.layer_norm_rows(rows, self.final_norm, self.final_bias, eps, dt)

    def _forward_shared_pre(self, input_ids, meta, ctx, caches: StackedCache) -> torch.Tensor:
        dt, eps, mult = self.dtype, self.cfg.rms_norm_eps, self.residual_mult
        if self.pair_embed is not None:
            table, mul_prev, mul_cur, buckets = self.pair_embed
            x = M.pair_embed_rows(input_ids, self.embed, self.embed_scale, table, mul_prev, mul_cur, buckets, ctx.seg,
                                  caches.extra["last_token"])
        else:
            x = M.embed_rows(input_ids, self.embed, self.embed_scale)
        tap, mark = self.layer_tap, self.mark_at
        nruns = len(self.runs)
        h = M.add_scaled_rms_norm_rows(x, None, None, mult, self.layers[self.runs[0][0]].norm1, eps, dt) \
            if nruns else None
        for r, (li, _) in enumerate(self.runs):
            if mark is not None and r == mark[0]:
                mark[1].record()
            L = self.layers[li]
            y = L.mixer(h, ctx, caches.per_run[r])
            f = L.ff(h, ctx) if L.ff is not None else None
            nw = self.layers[self.runs[r + 1][0]].norm1 if r + 1 < nruns else None
            h = M.add_scaled_rms_norm_rows(x, y, f, mult, nw, eps, dt)
            if tap is not None:
                tap.append(x.clone())
        idx = meta.logits_indices
        rows = x.index_select(0, idx) if idx.numel() != x.shape[0] else x
        if rows.shape[0] == 0:
            return rows.to(dt)
        return M.rms_norm_rows(rows, self.final_norm, eps, dt)

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        """fp32 logits [rows, vocab rounded up to a multiple of 8]; columns past the
        vocabulary are -inf.  With ``logit_softcap`` c > 0 the logits are c tanh(z / c)."""
        logits = self._head_product(h)
        if self.logit_scale != 1.0:
            logits *= self.logit_scale
        if self.logit_softcap:
            M.tanh_cap_(logits, self.logit_softcap)
        if self.vocab_pad:
            logits[:, self.cfg.vocab_size:] = float("-inf")
        return logits

    def _head_product(self, h: torch.Tensor) -> torch.Tensor:
        if h.dtype == torch.float32:
            return F.linear(h, self.head)
        # bf16 operands, fp32 accumulation and fp32 output
        if h.is_cuda and self._mm_out_dtype:
            try:
                return torch.mm(h, self.head.t(), out_dtype=torch.float32)
            except (TypeError, RuntimeError):
                self._mm_out_dtype = False   # this build has no fp32-output bf16 product
        return F.linear(h.float(), self.head.float())
