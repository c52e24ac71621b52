"""Kerarax: a decoder-only model of attention layers with no norm in front of the
sublayers -- each sublayer reads the residual itself, and a layer norm (weight and bias)
sits on its output: x += ln1(mixer(x)); x += ln2(ff(x)).

* Embedding: embed[token] plus a sinusoidal position vector over the whole width
  (column 2i: sin(p f_i), column 2i+1: cos(p f_i), f_i = 10000^(-2i/width)), then a layer
  norm (``embed.norm`` / ``embed.norm.b``).
* Mixer ``attention``: grouped-query attention whose q, k and v pass a short causal
  convolution right after their projections, per-head RMS norm of q and k with one
  shared weight vector each, no positions in the scores, scores capped by
  softcap tanh(s / softcap), every earlier key visible, and a softmax whose denominator
  has one added to it (:class:`..models.mixers.ConvSinkAttention`).
* Feed-forward (optional per layer): mixture of relu^2 experts; the ``top`` largest of
  the biased router logits are chosen and weighted by the softmax over just those; a
  shared expert runs for every token, scaled by a sigmoid gate
  (:class:`..models.mixers.MoEFF` with ``routing="top_logits"``, ``act="relu_sq"``).
* Output: layer norm (``final.norm`` / ``final.norm.b``), head, logits capped by
  logit_softcap tanh(z / logit_softcap).

Every size comes from ``config.json`` (keys: vocab, width, norm.eps, logit_softcap,
layers[].type / mixer{heads, kv_heads, dim, vdim, conv, scale, softcap} /
mlp{kind, router{experts, top}, expert{ff}, shared{ff}}) or from tensor shapes.  Tensor
names: embed, embed.norm(.b), head, final.norm(.b), l<i>.norm1(.b), l<i>.norm2(.b),
l<i>.mix.{q,k,v,o,q.conv,k.conv,v.conv,q.norm,k.norm},
l<i>.mlp.{router,router.b,e<j>.up,e<j>.down,shared.up,shared.down,shared.sg}.

The model body (layer runs, residual, caches, logits) is
:class:`..models.stacked.StackedModel` in its ``layer_post`` norm style.
"""
from __future__ import annotations

import dataclasses
import os
from typing import Dict, List, Optional, Tuple

import torch

from ..ops import mixers as M
from .mixers import ConvSinkAttention, MoEFF
from .registry import Architecture, register
from .stacked import StackedLayer, StackedModel

ATTENTION = "attention"
POSITION_BASE = 10000.0      # the design fixes the sinusoid's base
SINK_SCORE = 0.0             # and the score of the softmax's extra unit


@dataclasses.dataclass(frozen=True)
class KeraraxConfig:
    name: str
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float                # eps of every norm (layer norms and the per-head RMS norms)
    logit_softcap: float
    layers: tuple                      # per layer: dict(type=, mixer=, mlp=)
    max_position_embeddings: int = 1 << 17
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = False
    architecture = "kerarax"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> List[Tuple[int, Optional[int]]]:
        return [(i, None) for i in range(len(self.layers))]

    def num_params(self) -> int:
        return sum(int(torch.Size(s).numel()) for s in tensor_shapes(self).values())

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l["mixer"]["kv_heads"] * (l["mixer"]["dim"] + l["mixer"]["vdim"]) * dtype_bytes
                   for l in self.layers)


def config_from_dict(c: dict, name: str = "kerarax") -> KeraraxConfig:
    layers = []
    for i, l in enumerate(c["layers"]):
        if l["type"] != ATTENTION:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        m = dict(l["mixer"])
        m.setdefault("kv_heads", m["heads"])
        m.setdefault("vdim", m["dim"])
        m.setdefault("conv", 1)
        mlp = l.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            mlp = {"kind": "moe", "router": dict(mlp["router"]), "expert": dict(mlp["expert"]),
                   "shared": dict(mlp["shared"]) if mlp.get("shared") else None}
        layers.append({"type": ATTENTION, "mixer": m, "mlp": mlp})
    return KeraraxConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                         rms_norm_eps=float(c.get("norm", {}).get("eps", 1e-6)),
                         logit_softcap=float(c.get("logit_softcap") or 0.0), layers=tuple(layers),
                         max_position_embeddings=int(c.get("max_positions", 1 << 17)))


def config_to_dict(cfg: KeraraxConfig) -> dict:
    layers = []
    for l in cfg.layers:
        mlp = None
        if l["mlp"] is not None:
            mlp = {"kind": "moe", "router": dict(l["mlp"]["router"]), "expert": dict(l["mlp"]["expert"])}
            if l["mlp"]["shared"]:
                mlp["shared"] = dict(l["mlp"]["shared"])
        layers.append({"type": l["type"], "mixer": dict(l["mixer"]), "mlp": mlp})
    d = {"architecture": "Kerarax", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
         "norm": {"eps": cfg.rms_norm_eps}, "layers": layers}
    if cfg.logit_softcap:
        d["logit_softcap"] = cfg.logit_softcap
    return d


def tensor_shapes(cfg: KeraraxConfig) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration (random init, tests)."""
    w, v = cfg.hidden_size, cfg.vocab_size
    t: Dict[str, tuple] = {"embed": (v, w), "embed.norm": (w,), "embed.norm.b": (w,), "head": (v, w),
                           "final.norm": (w,), "final.norm.b": (w,)}
    for i, l in enumerate(cfg.layers):
        p, m = f"l{i}.", l["mixer"]
        h, g, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        t[p + "norm1"] = t[p + "norm1.b"] = (w,)
        t.update({p + "mix.q": (h * dk, w), p + "mix.k": (g * dk, w), p + "mix.v": (g * dv, w),
                  p + "mix.q.norm": (dk,), p + "mix.k.norm": (dk,), p + "mix.q.conv": (h * dk, taps),
                  p + "mix.k.conv": (g * dk, taps), p + "mix.v.conv": (g * dv, taps), p + "mix.o": (w, h * dv)})
        mlp = l["mlp"]
        if mlp is not None:
            t[p + "norm2"] = t[p + "norm2.b"] = (w,)
            e, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for j in range(e):
                t[p + f"mlp.e{j}.up"] = (ff, w)
                t[p + f"mlp.e{j}.down"] = (w, ff)
            t[p + "mlp.router"] = (e, w)
            t[p + "mlp.router.b"] = (e,)
            if mlp["shared"]:
                sf = mlp["shared"]["ff"]
                t.update({p + "mlp.shared.up": (sf, w), p + "mlp.shared.down": (w, sf), p + "mlp.shared.sg": (1, w)})
    return t


def random_tensors(cfg: KeraraxConfig, seed: int = 0, dtype=torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    """Random weights of the configuration's shapes: projections ~ N(0, 1/fan_in), norm
    weights near 1, small biases, convolution taps of order 1."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        r = torch.rand(shape, generator=g, device=device)
        n = torch.randn(shape, generator=g, device=device)
        if leaf == "conv":
            x = n * 0.5
        elif len(shape) == 2:
            x = n * (1.0 if name == "embed" else shape[1] ** -0.5)
        elif leaf == "b":
            x = 0.2 * n
        else:                                    # norm weights
            x = 0.75 + 0.5 * r
        out[name] = x.to(dtype)
    return out


def save_checkpoint(cfg: KeraraxConfig, tensors: Dict[str, torch.Tensor], out_dir: str):
    import json

    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.contiguous().cpu() for k, v in tensors.items()},
              os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(config_to_dict(cfg), f, indent=1)


class KeraraxModel(StackedModel):
    family = "Kerarax"
    norm_style = "layer_post"

    def load_tensors(self, get, has=lambda n: True):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        eps, width = cfg.rms_norm_eps, cfg.hidden_size
        self.load_head(get)
        nw = lambda n: self.norm_weight(get(n))   # noqa: E731
        self.embed_norm = (nw("embed.norm"), nw("embed.norm.b"))
        self.final_norm, self.final_bias = nw("final.norm"), nw("final.norm.b")
        self.pos_freqs = M.sinusoid_freqs(width, POSITION_BASE, device=dev)
        self.logit_softcap = cfg.logit_softcap
        self.layers = []
        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l["mixer"]
            mixer = ConvSinkAttention(lambda n, p=p: get(p + "mix." + n), width, m["heads"], m["kv_heads"],
                                      m["dim"], m["vdim"], m["conv"], m["scale"], m.get("softcap") or 0.0, eps,
                                      dt, dev, sink=SINK_SCORE)
            L = StackedLayer(l["type"], None, nw(p + "norm1"), mixer, bias1=nw(p + "norm1.b"))
            mlp = l["mlp"]
            if mlp is not None:
                L.norm2b, L.bias2 = nw(p + "norm2"), nw(p + "norm2.b")
                L.ff = MoEFF(lambda n, p=p: get(p + "mlp." + n), mlp["router"]["experts"], mlp["router"]["top"],
                             0.0, 1, 1, None, dt, dev, routing="top_logits", act="relu_sq",
                             shared=bool(mlp["shared"]))
            self.layers.append(L)
        return self

    def random_tensors(self, seed: int, device):
        return random_tensors(self.cfg, seed, torch.bfloat16, device=device)


# ---------------------------------------------------------------------------------------
# registry: shapes for random-init runs (benchmarks, smoke tests)
# ---------------------------------------------------------------------------------------

def _att(heads, kv_heads, dim, vdim, conv=4, softcap=30.0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
            "scale": dim ** -0.5, "softcap": softcap}


def _moe(experts, top, ff, shared_ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff},
            "shared": {"ff": shared_ff} if shared_ff else None}


def _preset(name, vocab, width, layers, cap=30.0):
    return config_from_dict({"vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "logit_softcap": cap,
                             "layers": layers}, name)


PRESETS = {
    # CPU-test sized
    "kerarax-tiny": _preset("kerarax-tiny", 320, 96, [
        {"type": ATTENTION, "mixer": _att(4, 2, 16, 24, conv=3, softcap=10.0), "mlp": _moe(6, 2, 48, 32)},
        {"type": ATTENTION, "mixer": _att(3, 1, 8, 8, conv=2, softcap=10.0), "mlp": None},
        {"type": ATTENTION, "mixer": _att(4, 4, 16, 16, conv=4, softcap=10.0), "mlp": _moe(4, 1, 64, 0)},
    ]),
    # a 2048-wide stack (benchmarks): 32 experts, top 4, and a shared expert; two matrices per
    # expert, sized so that a token's active expert weights equal those of nulazen-2k's
    # three-matrix experts (38 M per layer)
    "kerarax-2k": _preset("kerarax-2k", 32768, 2048, [
        {"type": ATTENTION, "mixer": _att(16, 4, 128, 128), "mlp": _moe(32, 4, 1536, 3072)} for _ in range(4)]),
    # the same stack at 4096 width (64 experts, top 6, as nulazen-4k)
    "kerarax-4k": _preset("kerarax-4k", 32768, 4096, [
        {"type": ATTENTION, "mixer": _att(32, 8, 128, 128), "mlp": _moe(64, 6, 2112, 4224)} for _ in range(4)]),
}


def _build(cfg, device, dtype, comm, max_model_len, quantization):
    return KeraraxModel(cfg, device, dtype, comm, max_model_len, quantization)


register(Architecture(
    name="kerarax",
    matches=lambda c: str(c.get("architecture", "")).lower() == "kerarax",
    parse=lambda c, name: config_from_dict(c, name),
    build=_build,
    presets=PRESETS,
))
