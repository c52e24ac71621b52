"""Shared cases of the Fufipel tests: small configurations with random weights, run
through the framework's engine (scheduler, block / state-slot pools, model runner,
kernels or the CPU backend) and compared with tests/fufipel_oracle.py.

None of the configurations is a real model's; they vary what a single model would leave
equal or 1: heads vs kv heads, key vs value sizes, value sizes over 64 and key sizes over
64, windows and blocks of one page, one page + 1, a single position, longer than the
prompt; kept first tokens none / fewer / more than a window; bias tables with an odd
number of rows; rotary dims none / part / all of a head, with and without the ramp; linear
attention with key sizes that are no multiple of 8 and value sizes over and under a 32
column tile; tau 1; residual and logit factors of 1; no pair table; layers without
feed-forward; borrowed keys and values once and twice; either mixer type first."""
import copy
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fufipel_oracle as O  # noqa: E402

from fasttalk_llm_microservice_amd.engine.config import EngineConfig  # noqa: E402
from fasttalk_llm_microservice_amd.engine.engine import LLMEngine  # noqa: E402
from fasttalk_llm_microservice_amd.models import fufipel as F  # noqa: E402


def _att(heads, kv, dim, vdim, window, keep, scale, rows, reach, kv_from=None):
    d = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": reach,
         "mask": {"size": window, "keep_first": keep}, "bias_rows": rows}
    if kv_from is not None:
        d["kv_from"] = kv_from
    return d


def _par(heads, kv, dim, vdim, block, scale, rot, lh, ldk, ldv, tau, rank):
    left = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": block}}
    if rot:
        left["rot"] = rot
    return {"left": left, "right": {"heads": lh, "dim": ldk, "vdim": ldv, "tau": tau, "rank": rank}}


def _rot(dims, base, scaling=None):
    d = {"dims": dims, "base": base}
    if scaling:
        d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return d


def _layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _cfg(vocab, width, eps, scale, mult, logit, bigram, layers):
    e = {"scale": scale}
    if bigram:
        e["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))
    return {"architecture": "Fufipel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": e,
            "residual_mult": mult, "logit_scale": logit, "layers": layers}


CONFIGS = {
    # attention first; window of one page + 1 with fewer kept tokens; a block of one page; part of each head
    # rotated with the ramp; two layers borrow one layer's keys and values; a layer without feed-forward
    "a": _cfg(101, 64, 1e-5, 3.0, 0.6, 1.5, (37, 5, 3), [
        _layer("attention", _att(4, 2, 8, 12, 17, 3, 0.3, 8, 40), 48),
        _layer("parallel", _par(4, 2, 12, 8, 16, 0.25, _rot(8, 1000.0, (4.0, 64, 4.0, 1.0)), 3, 10, 20, 4.0, 5), 40),
        _layer("attention", _att(4, 2, 8, 12, 9, 11, 0.35, 7, 30, kv_from=0), None),
        _layer("parallel", _par(2, 2, 16, 16, 33, 0.2, _rot(16, 500.0), 2, 8, 40, 12.0, 3), 24),
        _layer("attention", _att(4, 2, 8, 12, 30, 0, 0.3, 12, 100, kv_from=0), 32),
    ]),
    # parallel first; kv heads = heads; a value size over 64; no rotation at all; tau 1; factors of 1; no pair
    # table; a window of one position with kept tokens; a block longer than any prompt here
    "b": _cfg(77, 50, 1e-6, 1.0, 1.0, 1.0, None, [
        _layer("parallel", _par(2, 2, 6, 72, 1000, 0.4, None, 1, 12, 33, 1.0, 2), None),
        _layer("attention", _att(2, 2, 12, 72, 1, 4, 0.25, 6, 9), 20),
        _layer("parallel", _par(3, 1, 8, 8, 5, 0.3, _rot(4, 50.0, (2.0, 16, 2.0, 0.5)), 4, 8, 8, 2.0, 4), 36),
    ]),
    # a key size over 64; a window of exactly one page; a block of one position; everything kept first
    "c": _cfg(64, 40, 1e-5, 6.0, 0.25, 0.5, (7, 2, 9), [
        _layer("attention", _att(3, 1, 80, 16, 16, 0, 0.1, 9, 50), 28),
        _layer("parallel", _par(6, 2, 8, 24, 1, 0.3, _rot(8, 10000.0, (8.0, 32, 8.0, 2.0)), 2, 20, 64, 8.0, 6), 16),
        _layer("attention", _att(6, 3, 8, 8, 4, 64, 0.3, 5, 12), None),
    ]),
}


def make_model(name, seed, tmp_path, tweak=None):
    """(checkpoint dir, config dict, fp32 tensors of the bf16 weights)."""
    cfg = copy.deepcopy(CONFIGS[name])
    fcfg = F.config_from_dict(cfg, name)
    t = F.random_tensors(fcfg, seed, torch.bfloat16)
    if tweak:
        tweak(t)
    d = os.path.join(str(tmp_path), f"{name}-{seed}")
    F.save_checkpoint(fcfg, t, d)
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
    # bf16: rounding differs from the oracle's everywhere (the fp32 runs are the sharp ones)
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert err.median() < 0.06 and float(err.max()) < 0.25, err


def oracle(cfg, P, toks):
    return O.forward(cfg, P, toks).float()


def portions(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out
