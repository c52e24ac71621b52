"""Kerarax through the engine with the HIP kernels (fp32 sharp, bf16 loose) against the
plain oracle, each mechanism alone, greedy generation through LLMEngine.generate, and the
new kernels against the PyTorch implementation of the same op on multi-segment steps."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kerarax_cases as C  # noqa: E402
import kerarax_engine_cases as E  # noqa: E402
import kerarax_mechanism_cases as K  # noqa: E402

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


def test_peaked_and_flat_scores(tmp_path):
    E.peaked_and_flat_scores("cuda", "float32", tmp_path)


def test_long_decode(tmp_path):
    E.long_decode("cuda", "float32", tmp_path)


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

    d, cfg, _ = C.make_model("c", 3, tmp_path)
    eng = C.make_engine(d, "cuda", "bfloat16", seqs=3)
    outs = eng.generate([C.tokens(n, cfg["vocab"], n) for n in (3, 20, 1, 7)],
                        SamplingParams(temperature=0.8, top_p=0.9, max_tokens=9, ignore_eos=True, seed=1))
    assert [len(o) for o in outs] == [9] * 4 and all(0 <= t < cfg["vocab"] for o in outs for t in o)


def _segments(device, rows, pos0, slots, page, pad=0):
    """A step of several sequences (+ ``pad`` empty padding segments with slot -1)."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)   # noqa: E731
    start, tables, slot_map, nb = [0], [], [], 0
    maxb = max((p + r + page - 1) // page for p, r in zip(pos0, rows))
    for r, p in zip(rows, pos0):
        n = (p + r + page - 1) // page
        tab = list(range(nb, nb + n)) + [0] * (maxb - n)
        nb += n
        tables.append(tab)
        slot_map += [tab[q // page] * page + q % page for q in range(p, p + r)]
        start.append(start[-1] + r)
    kv = [p + r for p, r in zip(pos0, rows)]
    for _ in range(pad):
        start.append(start[-1])
        tables.append([0] * maxb)
        kv.append(0)
    seg = M.Segments(start=i32(start), pos0=i32(list(pos0) + [0] * pad), slot=i32(list(slots) + [-1] * pad),
                     kv_len=i32(kv), block_tables=i32(tables), num=len(rows) + pad, max_rows=max(rows), max_kv=max(kv))
    return seg, i32(slot_map), nb


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_prep_and_attention_kernels_multi_segment(dtype):
    """conv_attn_prep and the capped / sink attention kernel on a step of unequal segments
    (a decode row with history, a fresh prompt, a later portion, padding) against the
    PyTorch implementation of the same ops."""
    from fasttalk_llm_microservice_amd.ops import mixers as M
    from fasttalk_llm_microservice_amd.ops import mixers_ref as R

    g = torch.Generator().manual_seed(9)
    H, G, dk, dv, taps, page = 6, 2, 24, 40, 4, 8
    nq, nk, nv = H * dk, G * dk, G * dv
    rows, pos0, slots = [1, 13, 5, 1], [17, 0, 30, 2], [2, 0, 3, 1]
    seg, slot_map, nb = _segments("cuda", rows, pos0, slots, page, pad=2)
    T = sum(rows)
    qkv = (torch.randn(T, nq + nk + nv, generator=g) * 0.7).to("cuda", dtype)
    conv_w = (torch.randn(nq + nk + nv, taps, generator=g) * 0.5).cuda()
    wq, wk = (1 + 0.2 * torch.randn(dk, generator=g)).cuda(), (1 + 0.2 * torch.randn(dk, generator=g)).cuda()
    hist0 = torch.randn(4, taps - 1, nq + nk + nv, generator=g).cuda()
    kc0 = (torch.randn(nb, page, nk, generator=g) * 0.5).to("cuda", dtype)
    vc0 = (torch.randn(nb, page, nv, generator=g) * 0.5).to("cuda", dtype)
    outs = []
    for dev in ("cuda", "cpu"):
        mv = lambda t: t.clone().to(dev)   # noqa: E731
        sg = M.Segments(**{**seg.__dict__, **{k: getattr(seg, k).to(dev) for k in
                                              ("start", "pos0", "slot", "kv_len", "block_tables")}})
        hist, kc, vc = mv(hist0), mv(kc0), mv(vc0)
        q = M.conv_attn_prep(mv(qkv), nq, nk, mv(conv_w), hist, sg, mv(wq), mv(wk), 1e-5, dk, mv(slot_map), kc, vc)
        spec = M.WindowSpec(H, G, dk, dv, 0, 0.2, softcap=4.0, sink=0.0)
        o = M.window_attention(q, kc, vc, sg, spec)
        outs.append([t.float().cpu() for t in (q, hist, kc, vc, o)])
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for a, b, name in zip(outs[0], outs[1], ("q", "history", "k cache", "v cache", "attention")):
        torch.testing.assert_close(a, b, msg=lambda m, n=name: f"{n}: {m}", **tol)
    assert (outs[0][1][1] - hist0[1].cpu()).abs().max() > 0       # a one-row segment shifts its history


def test_graph_replays_of_new_kernels():
    """The layer norm, the fused convolution / norm / cache write and the capped attention
    inside a captured graph: several replays with eager work between them give what the
    eager calls give."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    g = torch.Generator().manual_seed(4)
    H, G, dk, dv, taps, page, W = 4, 2, 16, 16, 3, 8, 48
    nq, nk, nv = H * dk, G * dk, G * dv
    seg, slot_map, nb = _segments("cuda", [1, 1, 1], [5, 9, 1], [0, 2, 1], page, pad=1)
    qkv = torch.randn(3, nq + nk + nv, generator=g).cuda()
    conv_w = torch.randn(nq + nk + nv, taps, generator=g).cuda()
    wn = torch.ones(dk).cuda()
    w, b = torch.rand(W, generator=g).cuda(), torch.rand(W, generator=g).cuda()
    hist0 = torch.randn(3, taps - 1, nq + nk + nv, generator=g).cuda()
    kc0, vc0 = torch.randn(nb, page, nk, generator=g).cuda(), torch.randn(nb, page, nv, generator=g).cuda()
    x0, y = torch.randn(3, W, generator=g).cuda(), torch.randn(3, W, generator=g).cuda()
    spec = M.WindowSpec(H, G, dk, dv, 0, 0.25, softcap=5.0, sink=0.0)
    hist, kc, vc, x = hist0.clone(), kc0.clone(), vc0.clone(), x0.clone()

    def step():
        q = M.conv_attn_prep(qkv, nq, nk, conv_w, hist, seg, wn, wn, 1e-5, dk, slot_map, kc, vc)
        o = M.window_attention(q, kc, vc, seg, spec)
        M.add_layer_norm_rows(x, y, w, b, 1e-5, torch.float32)
        return o

    want_o = step().clone()
    want_x, want_h = x.clone(), hist.clone()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        hist.copy_(hist0); kc.copy_(kc0); vc.copy_(vc0); x.copy_(x0)
        step()
        s.synchronize()
        graph = torch.cuda.CUDAGraph()
        hist.copy_(hist0); x.copy_(x0)
        with torch.cuda.graph(graph, stream=s):
            out = step()
    for _ in range(3):
        hist.copy_(hist0); kc.copy_(kc0); vc.copy_(vc0); x.copy_(x0)
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(out, want_o, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(x, want_x, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(hist, want_h, rtol=0, atol=0)
        _ = (torch.randn(64, 64, device="cuda") @ torch.randn(64, 64, device="cuda")).sum().item()


@pytest.mark.parametrize("shape", [(70, 24, 20, 5), (333, 40, 100, 7), (1000, 256, 192, 16), (64, 64, 64, 1),
                                   (2048, 512, 136, 32)])
def test_grouped_product_kernel(shape):
    """The grouped expert product against one product per group: empty groups, groups that
    are no multiple of the row tile, N and K that are no multiples of the tile sizes."""
    from fasttalk_llm_microservice_amd.ops import mixers as M

    m, k, n, groups = shape
    g = torch.Generator().manual_seed(m + k)
    a = torch.randn(m, k, generator=g).to("cuda", torch.bfloat16)
    w = (torch.randn(groups, n, k, generator=g) * k ** -0.5).to("cuda", torch.bfloat16)
    flat = torch.randint(0, groups, (m,), generator=g)
    if groups > 2:
        flat[flat == 1] = 0                      # an empty group in the middle
        flat[flat == groups - 1] = 0             # and at the end
    counts = torch.bincount(flat, minlength=groups)
    offs = counts.cumsum(0).int().cuda()
    assert M.grouped_mm_is_one_product(a, w)
    got = M.grouped_mm(a, w, offs)
    want = torch.empty_like(got)
    s = 0
    for e, c in enumerate(counts.tolist()):
        want[s:s + c] = (a[s:s + c].float() @ w[e].float().t()).to(torch.bfloat16)
        s += c
    torch.testing.assert_close(got.float(), want.float(), rtol=1e-2, atol=1e-2)
    # fp32 rows take one product per group and give the same
    got32 = M.grouped_mm(a.float(), w.float(), offs)
    torch.testing.assert_close(got32, want.float(), rtol=1e-2, atol=1e-2)
