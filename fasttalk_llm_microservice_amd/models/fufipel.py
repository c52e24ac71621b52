"""Fufipel: a decoder-only model whose layers have ONE norm that both sublayers read, and
whose sublayer outputs are added together: h = norm1(x); x += residual_mult *
(mixer(h) + ff(h)).  Residual-stream norms store their weight as an offset from one
(x / rms(x) * (1 + w)).

* Embedding: embed[token] * embedding.scale plus an unscaled row of the pair table
  ``bigram``, chosen by (previous token * mul_prev + token * mul_cur) mod buckets; a
  sequence's first token takes row ``buckets``.  The previous token is part of a
  sequence's state (it lives in the sequence's state slot).
* Mixer ``attention``: grouped-query softmax attention without rotation, whole-projection
  RMS norms on q and k, a bias per head from a table over bucketed distances, a sliding
  window that also keeps the sequence's first tokens, a sigmoid output gate
  (:class:`..models.mixers.BiasedWindowAttention`).  With ``kv_from`` the layer has no
  keys and values of its own and reads the pages of the layer it names.
* Mixer ``parallel``: two mixers side by side on the same input
  (:class:`..models.mixers.SideBySide`) -- ``left``: attention with partly rotated heads
  (frequencies ramped down for long contexts) inside blocks of mask.size positions
  (:class:`..models.mixers.RotaryBlockAttention`); ``right``: linear attention with a decay
  per key channel (:class:`..models.mixers.GatedLinearAttention`).
* Feed-forward (optional per layer): down(relu(gate h) * (up h)).
* Output: the model's norm, then the embedding table itself as the head, times
  ``logit_scale``.

Every size comes from ``config.json`` (keys: vocab, width, norm.eps, residual_mult,
logit_scale, embedding{scale, bigram{buckets, mul_prev, mul_cur}}, layers[].type /
mixer / mlp{kind, ff}) or from tensor shapes.  Tensor names: embed, bigram, final.norm,
l<i>.norm1, l<i>.mix.{q,k,v,g,o,q.norm,k.norm,rel},
l<i>.mix.left.{q,k,v,o,out}, l<i>.mix.right.{q,k,v,g,o,norm,a1,a2,a2.b,out},
l<i>.mlp.{gate,up,down}.

The model body (layer runs, residual, caches, logits) is
:class:`..models.stacked.StackedModel` in its ``shared_pre`` norm style.
"""
from __future__ import annotations

import dataclasses
import os
from typing import Dict, List, Optional, Tuple

import torch

from .mixers import BiasedWindowAttention, GatedFF, GatedLinearAttention, RotaryBlockAttention, SideBySide
from .registry import Architecture, register
from .stacked import StackedLayer, StackedModel

ATTENTION, PARALLEL = "attention", "parallel"
PARALLEL_MEAN = 0.5          # the design fixes the weight of the two side-by-side outputs


@dataclasses.dataclass(frozen=True)
class FufipelConfig:
    name: str
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    embed_scale: float
    residual_mult: float
    logit_scale: float
    bigram: Optional[tuple]            # (buckets, mul_prev, mul_cur) or None
    layers: tuple                      # per layer: dict(type=, mixer=, mlp=)
    max_position_embeddings: int = 1 << 17
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = True
    architecture = "fufipel"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> List[Tuple[int, Optional[int]]]:
        return [(i, None) for i in range(len(self.layers))]

    def num_params(self) -> int:
        return sum(int(torch.Size(s).numel()) for s in tensor_shapes(self).values())

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        total = 0
        for l in self.layers:
            m = l["mixer"]["left"] if l["type"] == PARALLEL else l["mixer"]
            if m.get("kv_from") is None:
                total += m["kv_heads"] * (m["dim"] + m["vdim"]) * dtype_bytes
        return total


def _attention_sizes(m: dict) -> dict:
    m = dict(m)
    m.setdefault("kv_heads", m["heads"])
    m.setdefault("vdim", m["dim"])
    return m


def config_from_dict(c: dict, name: str = "fufipel") -> FufipelConfig:
    layers = []
    raw = c["layers"]
    for i, l in enumerate(raw):
        m = dict(l["mixer"])
        if l["type"] == ATTENTION:
            m = _attention_sizes(m)
            src = m.get("kv_from")
            if src is not None:
                src = int(src)
                o = raw[src]["mixer"] if 0 <= src < i and raw[src]["type"] == ATTENTION else None
                if o is None or o.get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
                o = _attention_sizes(o)
                if (o["kv_heads"], o["dim"], o["vdim"]) != (m["kv_heads"], m["dim"], m["vdim"]):
                    raise ValueError(f"layer {i}: kv_from names a layer with other key / value sizes")
                m["kv_from"] = src
        elif l["type"] == PARALLEL:
            m = {"left": _attention_sizes(m["left"]), "right": dict(m["right"])}
        else:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            mlp = {"kind": "dense", "ff": int(mlp["ff"])}
        layers.append({"type": l["type"], "mixer": m, "mlp": mlp})
    e = c.get("embedding", {})
    bg = e.get("bigram")
    return FufipelConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                         rms_norm_eps=float(c.get("norm", {}).get("eps", 1e-6)),
                         embed_scale=float(e.get("scale", 1.0)),
                         residual_mult=float(c.get("residual_mult", 1.0)),
                         logit_scale=float(c.get("logit_scale", 1.0)),
                         bigram=(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None,
                         layers=tuple(layers),
                         max_position_embeddings=int(c.get("max_positions", 1 << 17)))


def config_to_dict(cfg: FufipelConfig) -> dict:
    layers = []
    for l in cfg.layers:
        m = l["mixer"]
        m = {"left": dict(m["left"]), "right": dict(m["right"])} if l["type"] == PARALLEL else \
            {k: v for k, v in m.items() if v is not None}
        layers.append({"type": l["type"], "mixer": m, "mlp": dict(l["mlp"]) if l["mlp"] else None})
    emb = {"scale": cfg.embed_scale}
    if cfg.bigram:
        emb["bigram"] = {"buckets": cfg.bigram[0], "mul_prev": cfg.bigram[1], "mul_cur": cfg.bigram[2]}
    return {"architecture": "Fufipel", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "norm": {"eps": cfg.rms_norm_eps}, "embedding": emb, "residual_mult": cfg.residual_mult,
            "logit_scale": cfg.logit_scale, "layers": layers}


def tensor_shapes(cfg: FufipelConfig) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration (random init, tests)."""
    w, v = cfg.hidden_size, cfg.vocab_size
    t: Dict[str, tuple] = {"embed": (v, w), "final.norm": (w,)}
    if cfg.bigram:
        t["bigram"] = (cfg.bigram[0] + 1, w)
    for i, l in enumerate(cfg.layers):
        p, m = f"l{i}.", l["mixer"]
        t[p + "norm1"] = (w,)
        if l["type"] == ATTENTION:
            h, g, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": (h * dk, w), p + "mix.q.norm": (h * dk,), p + "mix.rel": (m.get("bias_rows", 32), h),
                      p + "mix.g": (h * dv, w), p + "mix.o": (w, h * dv)})
            if m.get("kv_from") is None:
                t.update({p + "mix.k": (g * dk, w), p + "mix.v": (g * dv, w), p + "mix.k.norm": (g * dk,)})
        else:
            a, b = m["left"], m["right"]
            h, g, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            t.update({p + "mix.left.q": (h * dk, w), p + "mix.left.k": (g * dk, w), p + "mix.left.v": (g * dv, w),
                      p + "mix.left.o": (w, h * dv), p + "mix.left.out": (w,), p + "mix.right.out": (w,)})
            h, dk, dv, r = b["heads"], b["dim"], b["vdim"], b.get("rank", 16)
            t.update({p + "mix.right.q": (h * dk, w), p + "mix.right.k": (h * dk, w), p + "mix.right.v": (h * dv, w),
                      p + "mix.right.g": (h * dv, w), p + "mix.right.o": (w, h * dv), p + "mix.right.norm": (dv,),
                      p + "mix.right.a1": (r, w), p + "mix.right.a2": (h * dk, r), p + "mix.right.a2.b": (h * dk,)})
        if l["mlp"] is not None:
            ff = l["mlp"]["ff"]
            t.update({p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return t


def random_tensors(cfg: FufipelConfig, seed: int = 0, dtype=torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    """Random weights of the configuration's shapes: projections ~ N(0, 1/fan_in),
    one-plus norm offsets near 0, plain norm weights near 1, decay biases that keep the
    recurrence lively."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        r = torch.rand(shape, generator=g, device=device)
        n = torch.randn(shape, generator=g, device=device)
        if name in ("embed", "bigram"):
            x = n
        elif leaf == "rel":
            x = 0.5 * n
        elif len(shape) == 2:
            x = n * shape[1] ** -0.5
        elif leaf == "b":
            x = 1.0 + 2.0 * r
        elif leaf == "norm1" or name == "final.norm":
            x = 0.25 * (r - 0.5)
        else:                                    # plain norm weights
            x = 0.75 + 0.5 * r
        out[name] = x.to(dtype)
    return out


def save_checkpoint(cfg: FufipelConfig, tensors: Dict[str, torch.Tensor], out_dir: str):
    import json

    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.contiguous().cpu() for k, v in tensors.items()},
              os.path.join(out_dir, "model.safetensors"))
    d = config_to_dict(cfg)
    for l in d["layers"]:                        # table sizes are tensor shapes, not configuration
        l["mixer"].pop("bias_rows", None)
        (l["mixer"].get("right") or {}).pop("rank", None)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(d, f, indent=1)


class FufipelModel(StackedModel):
    family = "Fufipel"
    norm_style = "shared_pre"

    def one_plus(self, t: torch.Tensor) -> torch.Tensor:
        """fp32 weight of a norm stored as an offset from one."""
        return (1.0 + self.norm_weight(t)).contiguous()

    def load_tensors(self, get, has=lambda n: True):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        eps, width = cfg.rms_norm_eps, cfg.hidden_size
        self.load_head(get, lambda n: n != "head" and has(n))     # the embedding table is the head
        self.embed_scale, self.logit_scale, self.residual_mult = cfg.embed_scale, cfg.logit_scale, cfg.residual_mult
        self.final_norm = self.one_plus(get("final.norm"))
        if cfg.bigram:
            buckets, mul_prev, mul_cur = cfg.bigram
            table = get("bigram").to(dev, dt).contiguous()
            if table.shape != (buckets + 1, width):
                raise ValueError("pair table does not fit its bucket count")
            self.pair_embed = (table, mul_prev, mul_cur, buckets)
        max_pos = max(self.max_model_len, 16) + 1
        self.layers = []
        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l["mixer"]
            if l["type"] == ATTENTION:
                mask = m.get("mask") or {}
                mixer = BiasedWindowAttention(
                    lambda n, p=p: get(p + "mix." + n), width, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                    int(mask.get("size", 0)), int(mask.get("keep_first", 0)), m["scale"], int(m["bias_max"]),
                    eps, dt, dev, cache_of=m.get("kv_from"))
            else:
                a, b = m["left"], m["right"]
                rot = a.get("rot") or {}
                sc = rot.get("scaling")
                left = RotaryBlockAttention(
                    lambda n, p=p: get(p + "mix.left." + n), width, a["heads"], a["kv_heads"], a["dim"], a["vdim"],
                    int((a.get("mask") or {}).get("size", 0)), a["scale"], int(rot.get("dims", 0)),
                    float(rot.get("base", 10000.0)),
                    (sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None, eps, dt, dev, max_pos)
                right = GatedLinearAttention(lambda n, p=p: get(p + "mix.right." + n), width, b["heads"], b["dim"],
                                             b["vdim"], b["tau"], eps, dt, dev)
                mixer = SideBySide(left, right, get(p + "mix.left.out"), get(p + "mix.right.out"), eps, dev,
                                   PARALLEL_MEAN)
            L = StackedLayer(l["type"], self.one_plus(get(p + "norm1")), None, mixer)
            if l["mlp"] is not None:
                L.ff = GatedFF(lambda n, p=p: get(p + "mlp." + n), dt, dev, act="relu")
            self.layers.append(L)
        return self

    def random_tensors(self, seed: int, device):
        return random_tensors(self.cfg, seed, torch.bfloat16, device=device)


# ---------------------------------------------------------------------------------------
# registry: shapes for random-init runs (benchmarks, smoke tests)
# ---------------------------------------------------------------------------------------

def _att(heads, kv_heads, dim, vdim, window, keep, kv_from=None, bias_rows=32, bias_max=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
         "mask": {"size": window, "keep_first": keep}, "bias_max": bias_max or 2 * window, "bias_rows": bias_rows}
    if kv_from is not None:
        d["kv_from"] = kv_from
    return d


def _par(heads, kv_heads, dim, vdim, block, lin_heads, lin_dim, lin_vdim, rot_dims=None, tau=8.0, rank=16,
         base=500000.0, scaling=True):
    rot = {"dims": rot_dims or dim, "base": base}
    if scaling:
        rot["scaling"] = {"factor": 8.0, "original": 8192, "fast": 24.0, "slow": 2.0}
    return {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                     "mask": {"size": block}, "rot": rot},
            "right": {"heads": lin_heads, "dim": lin_dim, "vdim": lin_vdim, "tau": tau, "rank": rank}}


def _preset(name, vocab, width, layers, scale=1.0, bigram=(4093, 1009, 917)):
    return config_from_dict({"vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.7,
                             "logit_scale": 1.0,
                             "embedding": {"scale": scale, "bigram": {"buckets": bigram[0], "mul_prev": bigram[1],
                                                                      "mul_cur": bigram[2]}},
                             "layers": layers}, name)


def _ff(n):
    return {"kind": "dense", "ff": n}


PRESETS = {
    # CPU-test sized
    "fufipel-tiny": _preset("fufipel-tiny", 320, 96, [
        {"type": PARALLEL, "mixer": _par(4, 2, 16, 24, 24, 3, 8, 16, rot_dims=8, rank=4), "mlp": _ff(128)},
        {"type": ATTENTION, "mixer": _att(4, 2, 16, 24, 20, 3, bias_rows=8, bias_max=30), "mlp": _ff(128)},
        {"type": ATTENTION, "mixer": _att(4, 2, 16, 24, 12, 2, kv_from=1, bias_rows=6, bias_max=20), "mlp": None},
    ], scale=4.0, bigram=(61, 7, 3)),
    # a 2048-wide stack (benchmarks): two side-by-side layers per attention layer, the last
    # attention layer on the first one's keys and values
    "fufipel-2k": _preset("fufipel-2k", 32768, 2048, [
        {"type": ATTENTION, "mixer": _att(16, 4, 128, 128, 1024, 64), "mlp": _ff(8192)},
        {"type": PARALLEL, "mixer": _par(16, 4, 128, 128, 1024, 16, 128, 128, rot_dims=64), "mlp": _ff(8192)},
        {"type": PARALLEL, "mixer": _par(16, 4, 128, 128, 1024, 16, 128, 128, rot_dims=64), "mlp": _ff(8192)},
        {"type": ATTENTION, "mixer": _att(16, 4, 128, 128, 1024, 64, kv_from=0), "mlp": _ff(8192)},
    ], scale=16.0),
    # the same stack at 4096 width
    "fufipel-4k": _preset("fufipel-4k", 32768, 4096, [
        {"type": ATTENTION, "mixer": _att(32, 8, 128, 128, 2048, 64), "mlp": _ff(14336)},
        {"type": PARALLEL, "mixer": _par(32, 8, 128, 128, 2048, 32, 128, 128, rot_dims=64), "mlp": _ff(14336)},
        {"type": PARALLEL, "mixer": _par(32, 8, 128, 128, 2048, 32, 128, 128, rot_dims=64), "mlp": _ff(14336)},
        {"type": ATTENTION, "mixer": _att(32, 8, 128, 128, 2048, 64, kv_from=0), "mlp": _ff(14336)},
    ], scale=16.0),
}


def _build(cfg, device, dtype, comm, max_model_len, quantization):
    return FufipelModel(cfg, device, dtype, comm, max_model_len, quantization)


register(Architecture(
    name="fufipel",
    matches=lambda c: str(c.get("architecture", "")).lower() == "fufipel",
    parse=lambda c, name: config_from_dict(c, name),
    build=_build,
    presets=PRESETS,
))
