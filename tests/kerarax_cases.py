"""Shared cases of the Kerarax tests: small configurations with random weights, run
through the framework's engine (scheduler, block / state-slot pools, model runner,
kernels or the CPU backend) and compared with tests/kerarax_oracle.py.

None of the configurations is a real model's; they vary what a single model would leave
equal or 1 (heads vs kv heads, key vs value sizes, one tap, several taps, a value size
over 64, a key size over 64, top 1, top = all experts, with and without a shared expert,
shared and expert sizes that differ, a layer without feed-forward first / in the middle,
layers of different sizes in one model, widths that are no multiple of 64)."""
import copy
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kerarax_oracle as O  # noqa: E402

from fasttalk_llm_microservice_amd.engine.config import EngineConfig  # noqa: E402
from fasttalk_llm_microservice_amd.engine.engine import LLMEngine  # noqa: E402
from fasttalk_llm_microservice_amd.models import kerarax as K  # noqa: E402


def _att(heads, kv, dim, vdim, conv, scale, softcap):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale, "softcap": softcap}


def _moe(experts, top, ff, shared_ff=None):
    d = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared_ff:
        d["shared"] = {"ff": shared_ff}
    return d


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


CONFIGS = {
    # layers of different sizes; a layer without feed-forward in the middle; top 1 without shared expert
    "a": {"architecture": "Kerarax", "vocab": 101, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 7.0,
          "layers": [_layer(_att(4, 2, 8, 12, 3, 0.3, 5.0), _moe(6, 2, 24, 40)),
                     _layer(_att(3, 1, 16, 10, 2, 0.2, 8.0), None),
                     _layer(_att(4, 4, 8, 8, 4, 0.35, 50.0), _moe(5, 1, 32))]},
    # kv heads = heads, one tap, every expert chosen, a value size over 64, no feed-forward first
    "b": {"architecture": "Kerarax", "vocab": 77, "width": 50, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
          "layers": [_layer(_att(2, 2, 12, 72, 1, 0.25, 3.0), None),
                     _layer(_att(2, 1, 6, 6, 2, 0.4, 12.0), _moe(3, 3, 20, 20))]},
    # a key size over 64, five taps, two experts
    "c": {"architecture": "Kerarax", "vocab": 64, "width": 40, "norm": {"eps": 1e-5}, "logit_softcap": 4.0,
          "layers": [_layer(_att(3, 1, 80, 16, 5, 0.1, 15.0), _moe(2, 1, 48, 8)),
                     _layer(_att(6, 2, 8, 24, 3, 0.3, 6.0), _moe(7, 3, 16, 56))]},
}


def make_model(name, seed, tmp_path, tweak=None):
    """(checkpoint dir, config dict, fp32 tensors of the bf16 weights)."""
    cfg = copy.deepcopy(CONFIGS[name])
    kcfg = K.config_from_dict(cfg, name)
    t = K.random_tensors(kcfg, seed, torch.bfloat16)
    if tweak:
        tweak(t)
    d = os.path.join(str(tmp_path), f"{name}-{seed}")
    K.save_checkpoint(kcfg, t, d)
    return d, cfg, {k: v.float() for k, v in t.items()}


def make_engine(ckpt, device, dtype="float32", pages=64, seqs=4, page=16, graphs=False):
    """``graphs``: decode steps replay captured graphs and are queued ahead (the
    serving configuration on a GPU); otherwise every step runs eagerly."""
    return LLMEngine(EngineConfig(model=ckpt, weights=ckpt, device=device, dtype=dtype, num_kv_blocks=pages,
                                  block_size=page, max_num_seqs=seqs, max_model_len=pages * page,
                                  max_num_batched_tokens=pages * page, enforce_eager=not graphs,
                                  async_output=graphs, swap_space_gb=0.0))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay(eng, reqs, schedule):
    """reqs: id -> tokens.  schedule: steps, each a list of (id, count).  Every position's
    logits are asked for.  Returns id -> [T, vocab] tensor."""
    at = {i: 0 for i in reqs}
    rows = {i: [] for i in reqs}
    for step in schedule:
        entries, end = [], []
        for i, n in step:
            lo, hi = at[i], at[i] + n
            entries.append((i, reqs[i][lo:hi], list(range(n))))
            at[i] = hi
            if hi == len(reqs[i]):
                end.append(i)
        lg = torch.from_numpy(eng.replay_step(entries, end).copy())
        k = 0
        for i, n in step:
            rows[i].append(lg[k:k + n])
            k += n
    return {i: torch.cat(v) for i, v in rows.items()}


def close(got, want, dtype="float32"):
    if dtype == "float32":
        torch.testing.assert_close(got, want, rtol=2e-4, atol=3e-4)
        return
    # bf16: rounding differs from the fp32 oracle everywhere; where two router logits are
    # closer than that rounding another expert is chosen and the row differs as a whole, so a
    # few rows may be off (the fp32 runs are the sharp ones)
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert err.median() < 0.08 and int((err > 0.3).sum()) <= max(1, err.numel() // 25), err


def oracle(cfg, P, toks):
    return O.forward(cfg, P, toks)


def portions(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out
