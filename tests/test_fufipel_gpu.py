"""Fufipel through the engine with the HIP kernels (fp32 sharp, bf16 loose) against the
plain oracle, each mechanism alone, greedy generation through LLMEngine.generate, and the
new kernels against the PyTorch implementation of the same op on multi-segment steps and
inside replayed graphs."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fufipel_cases as C  # noqa: E402
import fufipel_engine_cases as E  # noqa: E402
import fufipel_mechanism_cases as K  # noqa: E402

pytestmark = pytest.mark.gpu
CASES = [("a", "float32"), ("b", "float32"), ("c", "float32"), ("a", "bfloat16"), ("c", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompt(name, dtype, tmp_path):
    E.whole_prompt(name, "cuda", dtype, tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_layers(name, tmp_path):
    E.layers_of_a_prompt(name, "cuda", "float32", tmp_path)


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_then_decode(name, dtype, tmp_path):
    E.prefill_then_decode(name, "cuda", dtype, tmp_path)


@pytest.mark.parametrize("name", ["a", "c"])
def test_portions(name, tmp_path):
    E.portions_of_a_prompt(name, "cuda", "float32", tmp_path)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_and_reuse(name, dtype, tmp_path):
    E.mixed_batches_and_reuse(name, "cuda", dtype, tmp_path)


def test_peaked_scores(tmp_path):
    E.peaked_scores("cuda", "float32", tmp_path)


def test_slow_decay_long_decode(tmp_path):
    E.slow_decay_long_decode("cuda", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_greedy_generation(name, tmp_path):
    E.greedy_generation(name, "cuda", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_greedy_generation_graphs(name, tmp_path):
    """Decode steps replayed from captured graphs and queued ahead of the host."""
    E.greedy_generation(name, "cuda", "float32", tmp_path, graphs=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", K.CASES)
def test_mechanism(case, dtype):
    K.run(case, "cuda", dtype)


def test_bf16_generation_runs(tmp_path):
    from fasttalk_llm_microservice_amd.engine.sampling_params import SamplingParams

    d, cfg, _ = C.make_model("a", 3, tmp_path)
    eng = C.make_engine(d, "cuda", "bfloat16", seqs=3)
    outs = eng.generate([C.tokens(n, cfg["vocab"], n) for n in (3, 20, 1, 7)],
                        SamplingParams(temperature=0.8, top_p=0.9, max_tokens=9, ignore_eos=True, seed=1))
    assert [len(o) for o in outs] == [9] * 4 and all(0 <= t < cfg["vocab"] for o in outs for t in o)


def _segments(device, rows, pos0, slots, page, pad=0):
    """A step of several sequences (+ ``pad`` empty padding segments with slot -1)."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)   # noqa: E731
    start, tables, slot_map, nb, positions = [0], [], [], 0, []
    maxb = max((p + r + page - 1) // page for p, r in zip(pos0, rows))
    for r, p in zip(rows, pos0):
        n = (p + r + page - 1) // page
        tab = list(range(nb, nb + n)) + [0] * (maxb - n)
        nb += n
        tables.append(tab)
        slot_map += [tab[q // page] * page + q % page for q in range(p, p + r)]
        positions += list(range(p, p + r))
        start.append(start[-1] + r)
    kv = [p + r for p, r in zip(pos0, rows)]
    for _ in range(pad):
        start.append(start[-1])
        tables.append([0] * maxb)
        kv.append(0)
    seg = M.Segments(start=i32(start), pos0=i32(list(pos0) + [0] * pad), slot=i32(list(slots) + [-1] * pad),
                     kv_len=i32(kv), block_tables=i32(tables), num=len(rows) + pad, max_rows=max(rows), max_kv=max(kv))
    return seg, i32(slot_map), i32(positions), nb


def _on(seg, dev):
    from fasttalk_llm_microservice_amd.ops import mixers as M

    return M.Segments(**{**seg.__dict__, **{k: getattr(seg, k).to(dev) for k in
                                            ("start", "pos0", "slot", "kv_len", "block_tables")}})


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", ["window", "blocks"])
def test_attention_kernel_multi_segment(dtype, mask):
    """The per-row attention kernel with a block mask, or a window with kept first tokens and
    a distance table, on a step of unequal segments (decode rows deep in a sequence, a
    fresh prompt, a later portion, padding) against the PyTorch implementation."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    g = torch.Generator().manual_seed(9)
    H, G, dk, dv, page = 6, 2, 24, 40, 8
    nq, nk, nv = H * dk, G * dk, G * dv
    rows, pos0, slots = [1, 13, 5, 1], [70, 0, 30, 2], [2, 0, 3, 1]
    seg, slot_map, positions, nb = _segments("cuda", rows, pos0, slots, page, pad=2)
    T = sum(rows)
    qkv = (torch.randn(T, nq + nk + nv, generator=g) * 0.7).to("cuda", dtype)
    wq, wk = (1 + 0.2 * torch.randn(nq, generator=g)).cuda(), (1 + 0.2 * torch.randn(nk, generator=g)).cuda()
    kc0 = (torch.randn(nb, page, nk, generator=g) * 0.5).to("cuda", dtype)
    vc0 = (torch.randn(nb, page, nv, generator=g) * 0.5).to("cuda", dtype)
    rel = torch.randn(9, H, generator=g).cuda()
    table = M.rope_table(128, 16, 1000.0, device="cuda", ramp=(4.0, 64, 4.0, 1.0))
    outs = []
    for dev in ("cuda", "cpu"):
        mv = lambda t: t.clone().to(dev)   # noqa: E731
        sg = _on(seg, dev)
        kc, vc = mv(kc0), mv(vc0)
        if mask == "window":
            spec = M.WindowSpec(H, G, dk, dv, 11, 0.2, keep_first=5, dist_bias=M.distance_bias_table(mv(rel), 40))
            q = M.attn_prep(mv(qkv), nq, nk, mv(wq), mv(wk), 1e-5, None, 0, dk, mv(positions), mv(slot_map), kc, vc)
        else:
            spec = M.WindowSpec(H, G, dk, dv, 16, 0.2, blocks=True)
            q = M.attn_prep(mv(qkv), nq, nk, None, None, 1e-5, mv(table), 16, dk, mv(positions), mv(slot_map), kc, vc)
        o = M.window_attention(q, kc, vc, sg, spec)
        outs.append([t.float().cpu() for t in (q, kc, vc, o)])
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for a, b, name in zip(outs[0], outs[1], ("q", "k cache", "v cache", "attention")):
        torch.testing.assert_close(a, b, msg=lambda m, n=name: f"{n}: {m}", **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_kernels_multi_segment(dtype):
    """Pair-table embedding with slot state, gated linear attention, the gated head norm
    and the shared-norm add on a multi-segment step against the PyTorch implementation."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    g = torch.Generator().manual_seed(10)
    H, dk, dv, W, page = 3, 20, 40, 72, 8
    rows, pos0, slots = [1, 13, 5, 1], [17, 0, 30, 2], [2, 0, 3, 1]
    seg, _, _, _ = _segments("cuda", rows, pos0, slots, page, pad=2)
    T = sum(rows)
    ids = torch.randint(0, 50, (T,), generator=g).int()
    embed, pair = torch.randn(50, W, generator=g).to(dtype), torch.randn(12, W, generator=g).to(dtype)
    last0 = torch.tensor([9, 8, 7, 6], dtype=torch.int32)
    p = (torch.randn(T, H * (2 * dk + 2 * dv) + 5, generator=g) * 0.7).to(dtype)
    a = torch.randn(T, H * dk, generator=g).to(dtype)
    a_bias, norm_w = torch.randn(H * dk, generator=g) + 2.0, 1 + 0.2 * torch.randn(dv, generator=g)
    state0 = torch.randn(4, H, dk, dv, generator=g)
    y1, y2, nw = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g).to(dtype), torch.rand(W, generator=g)
    outs = []
    for dev in ("cuda", "cpu"):
        mv = lambda t: t.clone().to(dev)   # noqa: E731
        sg = _on(seg, dev)
        last, state = mv(last0), mv(state0)
        x = M.embed_rows(mv(ids), mv(embed), 3.0)
        M.pair_embed_add(x, mv(ids), mv(pair), 7, 5, 11, sg, last)
        o = M.gated_linear_attention(mv(p), mv(a), mv(a_bias), 8.0, state, sg, H, dk, dv)
        n0 = H * (2 * dk + dv)
        yg = M.head_rms_gate(o, mv(norm_w), mv(p)[:, n0:n0 + H * dv], 1e-5, H, dv, dtype, silu=True)
        h = M.add_scaled_rms_norm_rows(x, mv(y1), mv(y2), 0.5, mv(nw), 1e-5, dtype)
        outs.append([t.float().cpu() for t in (x, last, state, o, yg, h)])
    tol = dict(rtol=3e-5, atol=3e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for a_, b_, name in zip(outs[0], outs[1], ("residual", "last tokens", "state", "linear attention", "gated norm", "normed")):
        torch.testing.assert_close(a_, b_, msg=lambda m, n=name: f"{n}: {m}", **tol)
    assert outs[0][1].tolist() == [int(ids[13]), int(ids[19]), int(ids[0]), int(ids[18])]


def test_graph_replays_of_new_kernels():
    """Pair-table embedding, masked / biased attention, gated linear attention and the
    shared-norm add inside a captured graph: several replays with eager work between them
    give what the eager calls give."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    g = torch.Generator().manual_seed(4)
    H, G, dk, dv, page, W = 4, 2, 16, 16, 8, 48
    nq, nk, nv = H * dk, G * dk, G * dv
    seg, slot_map, positions, nb = _segments("cuda", [1, 1, 1], [25, 9, 1], [0, 2, 1], page, pad=1)
    ids = torch.tensor([4, 9, 2], dtype=torch.int32).cuda()
    embed, pair = torch.randn(12, W, generator=g).cuda(), torch.randn(8, W, generator=g).cuda()
    qkv = torch.randn(3, nq + nk + nv, generator=g).cuda()
    wq, wk = torch.ones(nq).cuda(), torch.ones(nk).cuda()
    spec = M.WindowSpec(H, G, dk, dv, 6, 0.25, keep_first=2,
                        dist_bias=M.distance_bias_table(torch.randn(6, H, generator=g).cuda(), 12))
    p, a = torch.randn(3, H * (2 * dk + dv), generator=g).cuda(), torch.randn(3, H * dk, generator=g).cuda()
    a_bias = torch.randn(H * dk, generator=g).cuda()
    y, nw = torch.randn(3, W, generator=g).cuda(), torch.rand(W, generator=g).cuda()
    kc0, vc0 = torch.randn(nb, page, nk, generator=g).cuda(), torch.randn(nb, page, nv, generator=g).cuda()
    st0, last0 = torch.randn(3, H, dk, dv, generator=g).cuda(), torch.tensor([3, 5, 7], dtype=torch.int32).cuda()
    kc, vc, st, last = kc0.clone(), vc0.clone(), st0.clone(), last0.clone()

    def step():
        x = M.embed_rows(ids, embed, 2.0)
        M.pair_embed_add(x, ids, pair, 3, 5, 7, seg, last)
        q = M.attn_prep(qkv, nq, nk, wq, wk, 1e-5, None, 0, dk, positions, slot_map, kc, vc)
        o = M.window_attention(q, kc, vc, seg, spec)
        l = M.gated_linear_attention(p, a, a_bias, 4.0, st, seg, H, dk, dv)
        h = M.add_scaled_rms_norm_rows(x, y, None, 0.5, nw, 1e-5, torch.float32)
        return o, l, h

    def reset():
        kc.copy_(kc0); vc.copy_(vc0); st.copy_(st0); last.copy_(last0)

    want = [t.clone() for t in step()]
    want_st, want_last = st.clone(), last.clone()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        reset()
        step()
        s.synchronize()
        graph = torch.cuda.CUDAGraph()
        reset()
        with torch.cuda.graph(graph, stream=s):
            out = step()
    for _ in range(3):
        reset()
        graph.replay()
        torch.cuda.synchronize()
        for got, w in zip(out, want):
            torch.testing.assert_close(got, w, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(st, want_st, rtol=1e-6, atol=1e-6)
        assert torch.equal(last, want_last)
        _ = (torch.randn(64, 64, device="cuda") @ torch.randn(64, 64, device="cuda")).sum().item()
