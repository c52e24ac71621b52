"""Each Kerarax mechanism of models/mixers.py (and the ops under it) alone against the
oracle's function for it: one whole sequence, then the same sequence cut in two steps
through the cache / state the first step left; with and without the matrix-product
attention path."""
import torch

import kerarax_oracle as O

from fasttalk_llm_microservice_amd.models import mixers as X
from fasttalk_llm_microservice_amd.ops import mixers as M

CASES = ["embedding", "layer_norm", "attention", "attention_products", "attention_product_chunks", "attention_one_tap_wide_value",
         "attention_long_taps", "attention_far_key", "attention_sink", "attention_cap", "router", "experts_pairs",
         "experts_sorted", "experts_all_chosen_no_shared", "logit_cap"]
EPS = 1e-5


def _rand(g, *shape, s=1.0):
    return (torch.randn(*shape, generator=g) * s).bfloat16().float()


def _ctx(T, device, cut=None, page=4, slot=1, host=False):
    """StepContexts of one sequence of T rows: whole, or [0, cut) then [cut, T)."""
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)   # noqa: E731
    nb = (T + page - 1) // page
    table = list(range(nb - 1, -1, -1))            # pages in reverse order
    out = []
    for a, b in ([(0, T)] if cut is None else [(0, cut), (cut, T)]):
        pos = list(range(a, b))
        seg = M.Segments(start=i32([0, b - a]), pos0=i32([a]), slot=i32([slot]), kv_len=i32([b]),
                         block_tables=i32([table]), num=1, max_rows=b - a, max_kv=b,
                         host=([0, b - a], [a], [b]) if host else None)
        slots = [table[p // page] * page + p % page for p in pos]
        out.append((a, b, X.StepContext(None, i32(pos), i32(slots), seg)))
    return out


def _close(got, want, dtype):
    """fp32: sharp.  bf16: rounding of the activations, measured against the output's size."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=3e-4, atol=3e-4)
    else:
        assert float((got - want).abs().max()) <= 0.05 * float(want.abs().max()) + 0.02


def _attention(device, dtype, host, T=45, H=4, G=2, dk=10, dv=7, taps=3, scale=0.3, cap=6.0,
               cuts=(None, 1, 2, 13, 36), tweak=None, rows=None, page=4):
    g = torch.Generator().manual_seed(3)
    W = 40
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "conv": taps, "scale": scale, "softcap": cap}
    P = {"q": _rand(g, H * dk, W, s=0.4), "k": _rand(g, G * dk, W, s=0.4), "v": _rand(g, G * dv, W, s=0.4),
         "q.conv": _rand(g, H * dk, taps, s=0.6), "k.conv": _rand(g, G * dk, taps, s=0.6),
         "v.conv": _rand(g, G * dv, taps, s=0.6), "q.norm": 1 + _rand(g, dk, s=0.2), "k.norm": 1 + _rand(g, dk, s=0.2),
         "o": _rand(g, W, H * dv, s=0.3)}
    h = _rand(g, T, W)
    if tweak:
        tweak(P, h)
    want = O.attention(m, P, "", h, EPS)
    mix = X.ConvSinkAttention(P.__getitem__, W, H, G, dk, dv, taps, scale, cap, EPS, dtype, device)
    for cut in cuts:
        cache = mix.alloc_cache((T + page - 1) // page, page, dtype, 3, device)
        cache[2].fill_(7.0)                         # a slot's old history is never read at position 0
        got = torch.cat([mix(h[a:b].to(device, dtype), ctx, cache).float().cpu()
                         for a, b, ctx in _ctx(T, device, cut, page=page, host=host)])
        _close(got if rows is None else got[rows], want if rows is None else want[rows], dtype)
        if taps > 1:
            assert float(cache[2][0].min()) == 7.0 and float(cache[2][2].max()) == 7.0   # other slots untouched
    return want


def _moe(device, dtype, T, experts, top, ff, shared_ff, W=24):
    g = torch.Generator().manual_seed(6)
    mlp = {"router": {"experts": experts, "top": top}, "expert": {"ff": ff},
           "shared": {"ff": shared_ff} if shared_ff else None}
    P = {"router": _rand(g, experts, W, s=0.6), "router.b": _rand(g, experts, s=0.5)}
    for j in range(experts):
        P[f"e{j}.up"] = _rand(g, ff, W, s=0.4)
        P[f"e{j}.down"] = _rand(g, W, ff, s=0.4)
    if shared_ff:
        P.update({"shared.up": _rand(g, shared_ff, W, s=0.4), "shared.down": _rand(g, W, shared_ff, s=0.4),
                  "shared.sg": _rand(g, 1, W, s=0.5)})
    h = _rand(g, T, W)
    ff_ = X.MoEFF(P.__getitem__, experts, top, 0.0, 1, 1, None, dtype, device, routing="top_logits", act="relu_sq",
                  shared=bool(shared_ff))
    got = ff_(h.to(device, dtype)).float().cpu()
    _close(got, O.moe(mlp, P, "", h), dtype)


def run(case, device, dtype):
    g = torch.Generator().manual_seed(1)
    if case == "embedding":
        for width in (20, 70):
            table = _rand(g, 11, width)
            w, b = 1 + _rand(g, width, s=0.2), _rand(g, width, s=0.2)
            toks = [3, 0, 10, 3, 7]
            cfg = {"width": width, "norm": {"eps": EPS}}
            want = O.embed(cfg, {"embed": table, "embed.norm": w, "embed.norm.b": b}, toks)
            # positions far from 0 too: the second half is a later portion of a long sequence
            for first in (0, 90000):
                pos = torch.arange(first, first + len(toks), dtype=torch.int32, device=device)
                x = M.embed_rows(torch.tensor(toks, dtype=torch.int32, device=device), table.to(device, dtype), 1.0,
                                 pos, M.sinusoid_freqs(width, 10000.0, device=device))
                if first == 0:
                    h = M.add_layer_norm_rows(x, None, w.to(device), b.to(device), EPS, dtype)
                    torch.testing.assert_close(x.cpu(), want, rtol=1e-5, atol=1e-5)
                    _close(h.float().cpu(), want, dtype)
                else:
                    sw = O.sinusoid(len(toks), width, first)
                    torch.testing.assert_close(x.cpu(), table[toks] + sw, rtol=0, atol=3e-2)   # fp32 angles at 9e4
    elif case == "layer_norm":
        for width in (24, 300):
            w, b = (1 + _rand(g, width, s=0.2)).to(device), _rand(g, width, s=0.2).to(device)
            x0 = _rand(g, 5, width) + 3.0
            y = (_rand(g, 5, width, s=4.0) - 2.0).bfloat16().float()                # means far from 0
            x = x0.clone().to(device)
            h = M.add_layer_norm_rows(x, y.to(device, dtype), w, b, EPS, dtype)
            want = x0 + O.layer_norm(y, w.cpu(), b.cpu(), EPS)
            torch.testing.assert_close(x.cpu(), want, rtol=1e-5, atol=1e-5)
            _close(h.float().cpu(), want, dtype)
            out = M.layer_norm_rows(x, w, b, EPS, dtype)
            torch.testing.assert_close(x.cpu(), want, rtol=1e-5, atol=1e-5)          # x itself is left alone
            _close(out.float().cpu(), O.layer_norm(want, w.cpu(), b.cpu(), EPS), dtype)
    elif case == "attention":
        _attention(device, dtype, host=False)
        _attention(device, dtype, host=False, H=3, G=3, dk=16, dv=16, taps=2, page=16)
    elif case == "attention_products":
        _attention(device, dtype, host=True, T=77, cuts=(None, 33, 40, 44))
        _attention(device, dtype, host=True, T=77, H=3, G=1, dk=16, dv=70, cuts=(None, 35))
    elif case == "attention_product_chunks":
        # a long segment is cut into chunks of rows; each sees the keys up to its own last row
        old = M.PRODUCT_FULL_CHUNK_ROWS, M.PRODUCT_SCORE_BYTES
        try:
            M.PRODUCT_FULL_CHUNK_ROWS = 40
            _attention(device, dtype, host=True, T=150, cuts=(None, 33, 100))
            M.PRODUCT_SCORE_BYTES = 4 * 4 * 35 * 150      # the memory bound halves the chunks again
            _attention(device, dtype, host=True, T=150, cuts=(None, 70))
        finally:
            M.PRODUCT_FULL_CHUNK_ROWS, M.PRODUCT_SCORE_BYTES = old
    elif case == "attention_one_tap_wide_value":
        _attention(device, dtype, host=False, H=2, G=2, dk=6, dv=72, taps=1)
    elif case == "attention_long_taps":
        # more taps than rows in the first portions: the history is shifted, not replaced
        _attention(device, dtype, host=False, T=30, taps=7, cuts=(None, 1, 2, 3, 6, 7, 29))
    elif case == "attention_far_key":
        # the first token's input is aligned with the last rows' and scaled up, and keys are made
        # from the query rows: the far key carries most of the weight among hundreds
        def tweak(P, h):
            P["k"].copy_(P["q"][:P["k"].shape[0]])
            P["k.conv"].copy_(P["q.conv"][:P["k.conv"].shape[0]])
            P["k.norm"].copy_(P["q.norm"])
            h[0:3] = h[-1] * 2.0
        for host in (False, True):
            _attention(device, dtype, host=host, T=230, H=2, G=2, taps=2, scale=1.0, cap=30.0, cuts=(None, 229, 100),
                       tweak=tweak, rows=slice(200, 230))
    elif case == "attention_sink":
        # tiny queries: all scores near 0, n keys weigh 1 / (n + 1) each
        def tweak(P, h):
            P["q.norm"] *= 0.01
        for host in (False, True):
            want = _attention(device, dtype, host=host, T=70, cuts=(None, 1, 40), tweak=tweak)
        assert want.abs().max() > 1e-2
    elif case == "attention_cap":
        # large queries: raw scores far above the cap, so the weights are those of capped scores
        def tweak(P, h):
            P["q.norm"] *= 8.0
        for host in (False, True):
            _attention(device, dtype, host=host, T=60, cap=2.5, cuts=(None, 33), tweak=tweak)
    elif case == "router":
        z = _rand(g, 9, 13)
        z[2, 5] = z[2, 1]                                 # a tie goes to the lower index
        for top in (1, 4, 13):
            idx, w = M.moe_top_logits(z.to(device), top)
            wi, ww = O.route(z, top)
            if top < 13:
                assert idx.cpu().long().tolist() == wi.tolist()
            torch.testing.assert_close(w.cpu(), ww, rtol=1e-5, atol=1e-6)
            assert torch.allclose(w.sum(-1).cpu(), torch.ones(9), atol=1e-5)
        # logits formed by the router kernel itself (few rows): widths with and without 16-byte rows
        for width in (64, 50, 7):
            h, rw, rb = _rand(g, 9, width), _rand(g, 13, width, s=0.5), _rand(g, 13, s=0.5)
            idx, w = M.moe_route_top_logits(h.to(device, dtype), rw.to(device), rb.to(device), 4)
            wi, ww = O.route(h @ rw.T + rb, 4)
            assert idx.cpu().long().tolist() == wi.tolist()
            torch.testing.assert_close(w.cpu(), ww, rtol=1e-4, atol=1e-5)
    elif case == "experts_pairs":
        _moe(device, dtype, 9, 6, 2, 20, 12)
    elif case == "experts_sorted":
        _moe(device, dtype, 70, 5, 2, 16, 24)
    elif case == "experts_all_chosen_no_shared":
        _moe(device, dtype, 5, 3, 3, 8, None)
        _moe(device, dtype, 66, 4, 1, 8, None)
    elif case == "logit_cap":
        x = _rand(g, 4, 16, s=20.0)
        x[1, 3] = float("-inf")
        got = M.tanh_cap_(x.clone().to(device), 9.0).cpu()
        want = O.capped(x, 9.0)
        assert got[1, 3] == float("-inf")
        want[1, 3] = float("-inf")
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
    else:
        raise KeyError(case)
