"""Engine-level Fufipel cases, run by tests/unit/test_fufipel_cpu.py (CPU backend) and
tests/test_fufipel_gpu.py (HIP kernels) with the device and dtype as arguments."""
import torch

import fufipel_cases as C
import fufipel_oracle as O

from fasttalk_llm_microservice_amd.engine.sampling_params import SamplingParams


def whole_prompt(name, device, dtype, tmp):
    d, cfg, P = C.make_model(name, 11, tmp)
    eng = C.make_engine(d, device, dtype)
    for n, seed in ((1, 1), (2, 2), (3, 3), (37, 4), (70, 5)):   # the first tokens, then longer prompts
        t = C.tokens(n, cfg["vocab"], seed)
        got = C.replay(eng, {"r": t}, [[("r", n)]])["r"]
        C.close(got, C.oracle(cfg, P, t), dtype)


def layers_of_a_prompt(name, device, dtype, tmp):
    """The residual after every layer against the oracle's."""
    d, cfg, P = C.make_model(name, 18, tmp)
    eng = C.make_engine(d, device, dtype)
    t = C.tokens(45, cfg["vocab"], 6)
    eng.runner.model.layer_tap = tap = []
    C.replay(eng, {"r": t}, [[("r", len(t))]])
    eng.runner.model.layer_tap = None
    want = O.layers(cfg, P, t)
    assert len(tap) == len(want)
    for g, w in zip(tap, want):
        torch.testing.assert_close(g.float().cpu(), w.float(), rtol=2e-4, atol=3e-4)


def prefill_then_decode(name, device, dtype, tmp):
    """Windows, blocks and kept tokens pass over decoded tokens; the pair table's previous
    token and the linear attention's state come from the step before."""
    d, cfg, P = C.make_model(name, 12, tmp)
    eng = C.make_engine(d, device, dtype)
    for first in (1, 2, 19, 40):
        t = C.tokens(first + 40, cfg["vocab"], 5 + first)
        sched = [[("r", first)]] + [[("r", 1)]] * 40
        C.close(C.replay(eng, {"r": t}, sched)["r"], C.oracle(cfg, P, t), dtype)


def portions_of_a_prompt(name, device, dtype, tmp):
    d, cfg, P = C.make_model(name, 13, tmp)
    eng = C.make_engine(d, device, dtype)
    t = C.tokens(115, cfg["vocab"], 9)
    want = C.oracle(cfg, P, t)
    # page size 16: cuts on and off page, window and block borders; 32+ rows take the
    # matrix-product attention, fewer the per-row kernel
    for sizes in ((2,), (1, 1, 1, 2, 3), (3, 2, 16, 1, 17, 5), (15, 1, 16, 17), (32, 2), (33, 41, 1, 40), (70, 45)):
        sched = [[("r", n)] for n in C.portions(len(t), sizes)]
        C.close(C.replay(eng, {"r": t}, sched)["r"], want, dtype)


def mixed_batches_and_reuse(name, device, dtype, tmp):
    """Unequal requests side by side (portions beside single tokens), more requests
    than state slots over time, a page pool smaller than the sum of all requests."""
    d, cfg, P = C.make_model(name, 14, tmp)
    eng = C.make_engine(d, device, dtype, pages=12, seqs=3)          # 192 tokens of cache, 3 slots
    lens = {"a": 70, "b": 9, "c": 41, "d": 1, "e": 55, "f": 30}
    reqs = {i: C.tokens(n, cfg["vocab"], 20 + k) for k, (i, n) in enumerate(lens.items())}
    sched = [
        [("a", 17), ("b", 1)],
        [("b", 1), ("a", 30), ("c", 5)],
        [("a", 1), ("b", 7), ("c", 1)],            # b ends: its slot and pages go back
        [("c", 33), ("a", 1), ("d", 1)],           # d takes b's slot; d ends
        [("a", 21), ("c", 1)],                     # a ends
        [("c", 1), ("e", 2), ("f", 16)],           # e, f reuse a's and d's slots and pages; c ends
        [("f", 1), ("e", 50)],
        [("e", 1), ("f", 13)],
        [("e", 1)],
        [("e", 1)],
    ]
    got = C.replay(eng, reqs, sched)
    for i, t in reqs.items():
        C.close(got[i], C.oracle(cfg, P, t), dtype)
    assert eng.scheduler.slots.num_free() == 3 and eng.bm.num_free() == 12
    # the same requests alone, one whole step each, give the same logits as in the batch
    if dtype == "float32":
        for i in ("a", "e"):
            alone = C.replay(eng, {i: reqs[i]}, [[(i, len(reqs[i]))]])[i]
            torch.testing.assert_close(alone, got[i], rtol=2e-4, atol=3e-4)


def peaked_scores(device, dtype, tmp):
    """Query norm weights and query projections scaled up: each row's weight sits on few
    keys anywhere it may look (far back among the kept first tokens, at a window's or a
    block's edge, at page borders), so a key lost or seen one position too far shows."""
    def tweak(t):
        for k in t:
            if k.endswith("mix.q.norm") or k.endswith("left.q"):
                t[k] *= 5.0
    for name in ("a", "c"):
        d, cfg, P = C.make_model(name, 15, tmp, tweak)
        eng = C.make_engine(d, device, dtype, pages=24)
        t = C.tokens(300, cfg["vocab"], 31)
        want = C.oracle(cfg, P, t)
        C.close(C.replay(eng, {"r": t}, [[("r", 250)]] + [[("r", 1)]] * 50)["r"], want, dtype)
        sched = [[("r", n)] for n in C.portions(300, (15, 17, 16, 1, 31, 33, 2, 100))]
        C.close(C.replay(eng, {"r": t}, sched)["r"], want, dtype)


def slow_decay_long_decode(device, dtype, tmp):
    """Decay biases raised so the linear attention's state fades slowly: 120 single-token
    steps after a three-token prompt carry it (and the previous token, and the caches)
    through every step; a state that is lost or reset shows."""
    def tweak(t):
        for k in t:
            if k.endswith("a2.b"):
                t[k] += 4.0
    d, cfg, P = C.make_model("c", 16, tmp, tweak)
    eng = C.make_engine(d, device, dtype)
    t = C.tokens(123, cfg["vocab"], 41)
    C.close(C.replay(eng, {"r": t}, [[("r", 3)]] + [[("r", 1)]] * 120)["r"], C.oracle(cfg, P, t), dtype)


def greedy_generation(name, device, dtype, tmp, graphs=False):
    """Through LLMEngine.generate: the scheduler's own batching, the sampler at
    temperature 0, against greedy decoding with the oracle."""
    d, cfg, P = C.make_model(name, 17, tmp)
    eng = C.make_engine(d, device, dtype, seqs=2, graphs=graphs)   # three prompts, two slots: one waits
    prompts = [C.tokens(n, cfg["vocab"], 50 + n) for n in (5, 1, 12)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True))
    for p, out in zip(prompts, outs):
        assert len(out) == 9
        seq = list(p)
        for tok in out:
            lg = O.forward(cfg, P, seq)[-1]
            best = int(lg.argmax())
            if best != tok:   # only a near-tie may differ
                assert lg[best] - lg[tok] < 1e-3, (seq, tok, best)
            seq.append(tok)
    assert eng.scheduler.slots.num_free() == 2
    if graphs:
        assert eng.runner.stats["graph_replays"] > 0
