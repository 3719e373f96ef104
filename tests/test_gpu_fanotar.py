"""The Fanotar decoder on the GPU against the plain implementation in tests/plain/fanotar.py: each
mechanism's kernel alone (with inputs made so that a fault shows: a far key whose score stands out, keys
just inside and just outside a window, at page borders, the first tokens where the sink weighs most, a
correction that changes which experts are chosen, sums beyond the gated unit's caps), then whole models
of four small configurations through trace replay (layer by layer, whole, token by token, in portions
down to two tokens, mixed batches on pages and state slots that are used again, long decoding), and
greedy generation through `LLM.generate` and the scheduler. float32 and bfloat16."""

from __future__ import annotations

import math

import pytest
import torch

from tests.helpers import fanotar_configs, prompt
from tests.plain import fanotar as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def hip():
    from tinyserve_llm_amd.ops import hip as h
    return h


def rounded(t: torch.Tensor, dtype: torch.dtype):
    """What the kernel gets: rounded to `dtype`; returns (device tensor, the same values in 64-bit on the host)."""
    d = t.to(dtype).to(DEV)
    return d, d.to(F64).cpu()


def tolerance(dtype):
    return dict(atol=5e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def step_context(tables, page, starts, counts, slots=None):
    """A packed step: request i feeds `counts[i]` tokens from position `starts[i]`, reads the pages
    `tables[i]` names and holds the state slot `slots[i]`."""
    from tinyserve_llm_amd.parts.base import StepContext
    positions, seq_of, cu = [], [], [0]
    for i, (s0, n) in enumerate(zip(starts, counts)):
        positions += list(range(s0, s0 + n))
        seq_of += [i] * n
        cu.append(cu[-1] + n)
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ends = [a + b for a, b in zip(starts, counts)]
    slots = list(range(len(starts))) if slots is None else list(slots)
    width = max(len(t) for t in tables)
    table = torch.tensor([list(t) + [0] * (width - len(t)) for t in tables], dtype=torch.int32, device=DEV)
    slot_map = [int(tables[i][p // page]) * page + p % page for i, (s0, n) in enumerate(zip(starts, counts)) for p in range(s0, s0 + n)]
    return StepContext(num_tokens=len(positions), num_seqs=len(starts), token_ids=dev([0] * len(positions)), positions=dev(positions),
                       seq_of_token=dev(seq_of), cu_seqlens=dev(cu), context_lens=dev(ends), state_slots=dev(slots),
                       slot_mapping=[dev(slot_map)], block_tables=[table], host_cu_seqlens=cu, host_starts=list(starts),
                       host_context_lens=ends, host_state_slots=slots, page_size=page)


def paged(pages: int, page: int, G: int, D: int, V: int, dtype):
    """A cache of its own for a kernel test: keys [pages, page, G, D], values kept transposed inside a
    page as the engine's pools keep them."""
    k = torch.zeros(pages, G, page, D, dtype=dtype, device=DEV).permute(0, 2, 1, 3)
    v = torch.zeros(pages, G, V, page, dtype=dtype, device=DEV).permute(0, 3, 1, 2)
    return k, v


# ---- the norm, the embedding, the gated unit ------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [80, 99, 256])
def test_dynamic_tanh_on_the_stream(dtype, width):
    h = hip()
    n = 7
    x = torch.randn(n, width) * 2
    a, a64 = rounded(torch.randn(n, width) * 3, dtype)
    norm = lambda: (torch.rand(1).to(DEV) + 0.2, (1 + 0.1 * torch.randn(width)).to(DEV), (0.1 * torch.randn(width)).to(DEV))
    post, pre = norm(), norm()
    f = lambda t, p: plain.dynamic_tanh(t, *(v.cpu().to(F64) for v in p))
    xd = x.to(DEV)
    out = h.dyt_stream(xd, a, post, pre, dtype)
    want = x.to(F64) + f(a64, post)
    torch.testing.assert_close(xd.cpu().to(F64), want, atol=2e-6, rtol=1e-6)
    torch.testing.assert_close(out.cpu().to(F64), f(want, pre), **tolerance(dtype))
    # a branch that is added as it is; the norm alone; picked rows in the order asked for, nothing updated
    before = xd.clone()
    assert h.dyt_stream(xd, a, None, None, dtype) is None
    torch.testing.assert_close(xd.cpu().to(F64), before.cpu().to(F64) + a64, atol=2e-6, rtol=1e-6)
    kept = xd.clone()
    alone = h.dyt_stream(xd, None, None, pre, dtype)
    assert torch.equal(xd, kept)
    torch.testing.assert_close(alone.cpu().to(F64), f(kept.cpu().to(F64), pre), **tolerance(dtype))
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    picked, _ = h.dyt(xd, *pre, dtype, rows=rows)
    torch.testing.assert_close(picked.cpu().to(F64), f(kept.cpu().to(F64)[[5, 0, 5]], pre), **tolerance(dtype))
    # plain rows with a residual: the sum comes back too
    r, r64 = rounded(torch.randn(n, width), dtype)
    y, total = h.dyt(a, *pre, dtype, residual=r, keep_sum=True)
    torch.testing.assert_close(total.cpu().to(F64), a64 + r64, **tolerance(dtype))
    torch.testing.assert_close(y.cpu().to(F64), f(total.cpu().to(F64), pre), **tolerance(dtype))


def test_embedding_scaled_and_normalised_into_the_stream():
    h = hip()
    table = torch.randn(50, 72).to(torch.bfloat16).to(DEV)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    norm = (torch.tensor([0.3], device=DEV), (1 + 0.1 * torch.randn(72)).to(DEV), (0.1 * torch.randn(72)).to(DEV))
    rows = table.cpu().to(F64)[[3, 49, 0, 3]] * 6.5
    got = h.embedding_dyt_stream(table, ids, 6.5, norm)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu().to(F64), plain.dynamic_tanh(rows, *(v.cpu().to(F64) for v in norm)), atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(h.embedding_dyt_stream(table, ids, 6.5).cpu().to(F64), rows, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_capped_gated_unit(dtype):
    h = hip()
    sums = torch.randn(9, 2 * 52) * 3                       # many beyond the caps on either side
    sums[0, :4] = torch.tensor([5.0, -5.0, 1.4999, 1.5001])
    sums[0, 52:56] = torch.tensor([9.0, -9.0, -1.5001, 1.4999])
    got = h.capped_glu(sums.to(DEV), 1.5, 1.702, 1.0, dtype)
    want = plain.capped_gated_unit(sums[:, :52].to(F64), sums[:, 52:].to(F64), 1.5)
    torch.testing.assert_close(got.cpu().to(F64), want, **(dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)))
    wide = torch.randn(4, 2 * 52 + 8)                       # rows that lie apart (a slice of a wider projection)
    got = h.capped_glu(wide.to(DEV)[:, :104], 0.8, 1.702, 1.0, torch.float32)
    torch.testing.assert_close(got.cpu().to(F64), plain.capped_gated_unit(wide[:, :52].to(F64), wide[:, 52:104].to(F64), 0.8), atol=1e-5, rtol=1e-5)


# ---- the short convolution, head norms, query multiplier, cache write, state -----------------------

CONV_SHAPES = [  # heads, kv heads (0: queries only), key size, value size, taps, query multiplier (coef, every)
    (4, 2, 32, 48, 3, (0.4, 4)),
    (2, 2, 16, 16, 5, (1.0, 3)),
    (6, 1, 24, 8, 1, (0.0, 1)),
    (3, 0, 20, 12, 4, (0.5, 2)),
    (8, 2, 64, 64, 4, (0.2, 32)),
    (1, 1, 200, 256, 2, (0.3, 5)),
]


@pytest.mark.parametrize("in_dtype, dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_convolution_norms_multiplier_cache_and_state(in_dtype, dtype, shape):
    """Three requests of unequal lengths fed in steps of unequal portions (single tokens, two tokens,
    portions shorter and longer than the taps reach back), in state slots that do not follow their order,
    one of which held another request before: q, the cached k and v rows and the state after every step
    equal the convolution over each request's whole sequence."""
    h = hip()
    H, G, D, V, taps, (coef, every) = shape
    C = (H + G) * D + G * V
    extra = 24                                              # (columns after the channels: a gate's)
    lengths, page = [300, 9, 281], 8                       # (a step of two long portions: its heads take the kernel of 16-byte pieces where they can, its values leave in tiles)
    conv = (torch.randn(C, taps) * 0.4 + 1.0 / taps).to(DEV)
    qn, kn = (1 + 0.2 * torch.randn(D)).to(DEV), (1 + 0.2 * torch.randn(D)).to(DEV)
    proj = [rounded(torch.randn(n, C + extra), in_dtype) for n in lengths]
    pages = [-(-n // page) for n in lengths]
    order = torch.randperm(sum(pages) + 2).tolist()
    tables = [order[sum(pages[:i]):sum(pages[:i + 1])] for i in range(3)]
    k, v = paged(sum(pages) + 2, page, max(G, 1), D, V, dtype)
    slots = [2, 0, 3]
    state = torch.randn(4, taps - 1, C, device=DEV) if taps > 1 else None      # what a request before left behind
    if taps > 1:
        for s in slots:
            state[s].zero_()                                # (a slot is cleared when a request takes it)
    want_q, want_k, want_v = [], [], []
    eps = 1e-5
    for (_, p64), n in zip(proj, lengths):
        y = plain.short_convolution(p64[:, :C], conv.cpu().to(F64))
        q = plain.unit_rms(y[:, :H * D].view(n, H, D), eps) * qn.cpu().to(F64)
        q = q * plain.query_multiplier(torch.arange(n, dtype=F64), coef, every)[:, None, None] if coef else q
        want_q.append(q)
        if G:
            want_k.append(plain.unit_rms(y[:, H * D:(H + G) * D].view(n, G, D), eps) * kn.cpu().to(F64))
            want_v.append(y[:, (H + G) * D:].view(n, G, V))
    cuts = [[1, 2, 1, 2, 2, 292], [2, 1, 1, 1, 4], [7, 1, 1, 12, 3, 257]]      # (the first long portion starts at a page's first slot, the second does not)
    cursors, got_q = [0, 0, 0], [[], [], []]
    for step in range(max(len(c) for c in cuts)):
        live = [i for i in range(3) if step < len(cuts[i])]
        counts = [cuts[i][step] for i in live]
        starts = [cursors[i] for i in live]
        ctx = step_context([tables[i] for i in live], page, starts, counts, [slots[i] for i in live])
        rows = torch.cat([proj[i][0][cursors[i]:cursors[i] + cuts[i][step]] for i in live])
        q = h.conv_finish(rows, conv, state, ctx, ctx.slot_mapping[0] if G else None, k if G else None, v if G else None, H, G, D, V,
                          dtype, q_norm=qn, k_norm=kn if G else None, eps=eps, temp_coef=coef, temp_every=every,
                          moves_state=(fused := taps > 1 and h.conv_moves_state(ctx)))
        assert fused == (taps > 1 and set(counts) == {1})     # (the third step: a token of each request)
        if taps > 1 and not fused:
            h.conv_state_update(state, rows, ctx)
        at = 0
        for i, n in zip(live, counts):
            got_q[i].append(q[at:at + n])
            at += n
            cursors[i] += n
            if taps > 1:
                # the state: the last taps - 1 projected rows so far, zeros before the request's start
                seen = proj[i][1][:cursors[i], :C]
                want = torch.cat([torch.zeros(taps - 1, C, dtype=F64), seen])[-(taps - 1):]
                torch.testing.assert_close(state[slots[i]].cpu().to(F64), want, atol=0, rtol=0)
    assert cursors == lengths
    tol = tolerance(dtype)
    for i in range(3):
        torch.testing.assert_close(torch.cat(got_q[i]).cpu().to(F64), want_q[i], **tol)
        for p in range(lengths[i] if G else 0):
            pg = tables[i][p // page]
            torch.testing.assert_close(k[pg, p % page].cpu().to(F64), want_k[i][p], **tol)
            torch.testing.assert_close(v[pg, p % page].cpu().to(F64), want_v[i][p], **tol)


# ---- attention with slopes, learned sinks, a window and a gate --------------------------------------

def attention_case(dtype, H, G, D, V, page, length, queries, stand_out, scale, window, gate=True, seed=0, sink_value=None,
                   portion_from=None):
    """Keys and values of one request of `length` tokens on shuffled pages, queries at the positions
    `queries`, each a decoded token of a request of its own over the same pages; with `portion_from`, one
    request instead that feeds the positions from there to the end as one portion of a prompt (0: the whole
    prompt), every position a query. `stand_out` maps a query's position to the key position whose score is
    made to stand out for it (the key is set to a multiple of the query's direction that outweighs the
    distance penalty of the steepest head). Returns (kernel output, oracle output, values, query positions)."""
    h = hip()
    if portion_from is not None:
        queries = list(range(portion_from, length))
        stand_out = {q: key for q, key in stand_out.items() if q >= portion_from}
    gen = torch.Generator().manual_seed(seed)
    k64 = plain.unit_rms(torch.randn(length, G, D, generator=gen, dtype=F64), 0.0)
    v64 = torch.randn(length, G, V, generator=gen, dtype=F64)
    q64 = plain.unit_rms(torch.randn(len(queries), H, D, generator=gen, dtype=F64), 0.0)
    slopes = plain.distance_slopes(H)
    for i, p in enumerate(queries):
        if p in stand_out:
            g_dir = plain.unit_rms(torch.randn(G, D, generator=gen, dtype=F64), 0.0)
            for hh in range(H):
                q64[i, hh] = g_dir[hh // (H // G)]
            # q.k * scale = boost * D * scale: 8 above what the distance takes off
            k64[stand_out[p]] = (8.0 + slopes[0] * (p - stand_out[p])) / (D * scale) * g_dir
    sinks = torch.randn(H, generator=gen, dtype=F64) if sink_value is None else torch.full((H,), sink_value, dtype=F64)
    gates = torch.randn(len(queries), H * V, generator=gen) * 2
    pages = -(-length // page)
    table = torch.randperm(pages + 3, generator=gen)[:pages].tolist()
    k, v = paged(pages + 3, page, G, D, V, dtype)
    kr, vr = k64.to(dtype), v64.to(dtype)
    for p in range(length):
        k[table[p // page], p % page] = kr[p].to(DEV)
        v[table[p // page], p % page] = vr[p].to(DEV)
    q = q64.to(dtype).to(DEV)
    if portion_from is None:
        ctx = step_context([table] * len(queries), page, queries, [1] * len(queries))
    else:
        ctx = step_context([table], page, [portion_from], [len(queries)])
    wide = torch.cat([torch.zeros(len(queries), 5), gates], 1).to(DEV)          # (the gate: columns of a wider row)
    out = h.paged_attention(q, k, v, ctx, 0, scale, window, sinks=sinks.float().to(DEV),
                            slopes=torch.tensor(slopes, dtype=torch.float32, device=DEV), gate=wide[:, 5:] if gate else None)
    want = plain.sloped_sink_attention(q.cpu().to(F64), kr.to(F64), vr.to(F64), torch.tensor(queries), scale, slopes,
                                       sinks.float().to(F64), window)
    if gate:
        want = want * torch.sigmoid(gates.to(F64)).view(len(queries), H, V)
    return out.cpu().to(F64), want, vr.to(F64), queries


FORMS = {"decoded": None, "prompt": 0, "portion": 130}       # (a portion that starts inside a page)


@pytest.mark.parametrize("form", sorted(FORMS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 32, 48), (2, 2, 16, 16), (6, 1, 24, 8), (8, 2, 64, 64), (4, 4, 128, 128)])
def test_attention_far_keys_page_borders_and_first_tokens(dtype, sizes, form):
    H, G, D, V = sizes
    page, length = 16, 700
    # no window: a key hundreds of tokens back, keys at both sides of page borders, the query's own key, the first tokens
    stand_out = {699: 3, 650: 15, 651: 16, 652: 17, 653: 653, 500: 255, 501: 256, 31: 0}
    queries = [0, 1, 2, 3, 15, 16, 17, 31, 500, 501, 650, 651, 652, 653, 699]
    out, want, v, queries = attention_case(dtype, H, G, D, V, page, length, queries, stand_out, D ** -0.5, 0, gate=False,
                                           portion_from=FORMS[form])
    torch.testing.assert_close(out, want, **tolerance(dtype))
    i = queries.index(699)
    assert float((want[i, 0] - v[3, 0]).abs().max()) < 0.2 * float(v[3, 0].abs().max()), "the far key decides the row"
    out, want, _, _ = attention_case(dtype, H, G, D, V, page, 90, [0, 1, 5, 17, 89], {89: 2}, 0.9 / D ** 0.5, 0, gate=True, seed=1,
                                     portion_from=None if FORMS[form] is None else FORMS[form] // 10)
    torch.testing.assert_close(out, want, **tolerance(dtype))


@pytest.mark.parametrize("form", sorted(FORMS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window, sizes", [(1, (4, 2, 32, 40)), (7, (4, 2, 32, 40)), (16, (4, 2, 32, 40)), (40, (4, 2, 32, 40)),
                                           (64, (4, 2, 32, 40)), (100, (4, 2, 32, 40)), (7, (4, 2, 64, 64)), (65, (4, 2, 64, 64)),
                                           (130, (4, 1, 64, 64)), (33, (2, 2, 128, 128)), (257, (6, 2, 32, 32))])
def test_attention_window_edges(dtype, window, sizes, form):
    """The key that stands out lies just inside the window for some queries and just outside for others
    (then it must not count at all), at windows shorter and longer than a page, than a wave's chunk of keys and
    than a matrix-core tile, for decoded tokens, a whole prompt and a portion of one."""
    (H, G, D, V), page, length = sizes, 16, 600
    # (the queries with a key that stands out lie further apart than the widest window, so that none sees another's)
    if window > 100:
        length = 4 * window + 15
        inside = {q: q - window + 1 for q in (window - 1, 3 * window + 9)}
        outside = {q: q - window for q in (2 * window + 4, 4 * window + 14)}
    else:
        inside = {q: q - window + 1 for q in (window - 1, 400)}
        outside = {q: q - window for q in (200, 599)}
    queries = sorted({0, 127, 128, 129, *inside, *outside})
    out, want, v, queries = attention_case(dtype, H, G, D, V, page, length, queries, {**inside, **outside}, D ** -0.5, window,
                                           gate=False, sink_value=-3.0, portion_from=FORMS[form])
    torch.testing.assert_close(out, want, **tolerance(dtype))
    # the test is sharp: an inside key decides its row, an outside key leaves the row to the others
    for q, key in inside.items():
        if q in queries:
            i = queries.index(q)
            assert float((want[i, 0] - v[key, 0]).abs().max()) < 0.2 * float(v[key, 0].abs().max())
    for q, key in outside.items():
        if q in queries and window > 1:
            i = queries.index(q)
            assert float((want[i, 0] - v[key, 0]).abs().max()) > 0.2 * float(v[key, 0].abs().max())


def test_the_sink_weighs_most_on_the_first_tokens():
    # a large learned sink takes nearly all the weight where there are few keys: the output is small there
    out, want, v, _ = attention_case(torch.float32, 4, 2, 32, 32, 16, 40, [0, 1, 39], {}, 32 ** -0.5, 0, gate=False, sink_value=6.0)
    torch.testing.assert_close(out, want, atol=2e-5, rtol=1e-5)
    assert float(out[0].abs().max()) < 0.02 * float(v[0].abs().max())


# ---- the router and the experts --------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(6, 3, 80, 40, 23), (4, 1, 48, 20, 1), (5, 5, 99, 17, 9), (12, 2, 64, 24, 70), (8, 2, 512, 128, 40),
                                   (4, 2, 64, 32, 170), (3, 1, 96, 160, 300), (3, 2, 128, 192, 300), (2, 1, 192, 64, 513)])
def test_router_grouping_and_experts(dtype, sizes):
    h = hip()
    E, top, W, F, n = sizes
    x, x64 = rounded(torch.randn(n, W), dtype)
    router = (torch.randn(E, W) * 0.3).to(DEV)
    corr = torch.randn(E).to(DEV)                            # (of the size of the scores: it changes who is chosen)
    ids, weights = h.moe_route(x, router, corr, top, 1.7)
    z = x64 @ router.cpu().to(F64).T
    chosen, w64 = plain.route(z, corr.cpu().to(F64), top, 1.7)
    for t in range(n):
        # no close calls are made: where the oracle's margin is wide the choice is the same
        c = torch.sigmoid(z[t]) + corr.cpu().to(F64)
        ranked = torch.sort(c, descending=True).values
        if top < E and float(ranked[top - 1] - ranked[top]) < 1e-3:
            continue
        assert sorted(ids[t].tolist()) == sorted(chosen[t].tolist())
        got = dict(zip(ids[t].tolist(), weights[t].tolist()))
        for e, w in zip(chosen[t].tolist(), w64[t].tolist()):
            assert got[e] == pytest.approx(w, rel=1e-4, abs=1e-5)
    # the experts on the engine's own choice
    gate_up, gu64 = rounded(torch.randn(E, 2 * F, W) * W ** -0.5 * 2, dtype)
    down, d64 = rounded(torch.randn(E, W, F) * F ** -0.5, dtype)
    # (the last two cases give an expert enough rows for the wide tiles of the matrix-core kernel in bfloat16)
    tile_rows = h.moe_tile_rows(n * top, E, dtype, (W, F))
    # (the last cases give an expert enough rows for the tiles of 64 and of 128 rows in bfloat16)
    wide = 16 if dtype != torch.bfloat16 or n < 170 else 128 if n * top >= 128 * E and W % 64 == 0 and F % 64 == 0 else 64
    assert tile_rows == wide
    grouped = h.moe_group(ids, E, tile_rows)
    tiles = grouped.tiles.cpu()
    assert sorted(grouped.sorted.cpu().tolist()) == list(range(n * top))
    assert int(tiles[:, 2].sum()) == n * top and int(tiles[:, 2].max()) <= tile_rows
    for e, first, rows in tiles.tolist():
        assert all(int(ids.view(-1)[p]) == e for p in grouped.sorted[first:first + rows].tolist())
    unit = h.moe_gemm(x, gate_up, grouped, dtype, per_token=True, glu=(1.2, 1.702, 1.0))
    rows = h.moe_gemm(unit, down, grouped, torch.float32, per_token=False)
    shared = torch.randn(n, W).to(DEV)
    out = h.moe_combine(rows, weights, shared)
    want = shared.cpu().to(F64).clone()
    flat = ids.cpu().view(-1).tolist()
    for t in range(0, n, max(1, n // 40)):
        for j in range(top):
            e = flat[t * top + j]
            y = plain.capped_gated_unit(x64[t] @ gu64[e, :F].T, x64[t] @ gu64[e, F:].T, 1.2)
            torch.testing.assert_close(unit[t * top + j].cpu().to(F64), y, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)))
            want[t] += float(weights[t, j]) * (unit[t * top + j].cpu().to(F64) @ d64[e].T)
    picked = list(range(0, n, max(1, n // 40)))
    out, want = out[picked], want[picked]
    torch.testing.assert_close(out.cpu().to(F64), want, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)))


# ---- whole models through trace replay ---------------------------------------------------------------

LENGTHS = {"P": [1, 23, 97, 200], "Q": [1, 30, 75, 150], "R": [2, 19, 66, 131], "S": [1, 40, 140]}
TOL = {"float32": 2e-4, "bfloat16": 6e-2}       # of the spread of the oracle's logits


@pytest.fixture(scope="module", params=["P", "Q", "R", "S"])
def case(request, tmp_path_factory):
    from tinyserve_llm_amd.weights.random_init import write_random_model
    name = request.param
    config, seed = fanotar_configs()[name]
    folder = str(tmp_path_factory.mktemp(f"fanotar_{name}"))
    write_random_model(folder, config, seed, torch.bfloat16)
    oracle = plain.PlainFanotar(folder)
    prompts = [prompt(500 + i, n, config.vocab) for i, n in enumerate(LENGTHS[name])]
    return name, folder, config, prompts, oracle, [oracle.logits(p) for p in prompts]


def replayer(folder, dtype, max_tokens):
    from tinyserve_llm_amd.engine.replay import Replay
    return Replay(folder, dtype, max_tokens)


def check(got, oracle_rows, dtype):
    assert got, "nothing was compared"
    spread = float(torch.cat([o.flatten() for o in oracle_rows]).std())
    worst = 0.0
    for (r, pos), row in got.items():
        want = oracle_rows[r][pos]
        torch.testing.assert_close(row.double().cpu(), want, atol=TOL[dtype] * spread, rtol=0.0,
                                   msg=lambda m: f"request {r} position {pos}: {m}")
        worst = max(worst, float((row.double().cpu() - want).abs().max()))
    print(f"[{dtype}] worst logit error {worst / spread:.3e} of the logits' spread ({spread:.2f}) over {len(got)} rows")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_streams_and_whole_requests(case, dtype):
    name, folder, config, prompts, oracle, rows = case
    rep = replayer(folder, dtype, 256)
    got = {}
    for r, p in enumerate(prompts):
        logits = rep.step([{"id": f"r{r}", "tokens": p, "want": list(range(len(p)))}], [f"r{r}"])
        assert logits.shape == (len(p), config.vocab) and logits.dtype == torch.float32
        for pos in range(len(p)):
            got[(r, pos)] = logits[pos]
    check(got, rows, dtype)
    assert rep.manager.num_available_blocks() == rep.manager.num_blocks, "every page came back"
    assert len(rep.manager.free_state_slots) == 4, "every state slot came back"
    if dtype == "float32":
        # the residual stream after every layer, layer by layer
        from tinyserve_llm_amd.engine.runner import StepEntry
        from tinyserve_llm_amd.parts import base
        from tinyserve_llm_amd.parts.stream import ResidualStream
        p = prompts[2]
        want = oracle.streams(p)
        rep.manager.allocate(77, p)
        ctx, _, _ = rep.runner.prepare([StepEntry(77, p, 0, [])])
        hidden, residual = rep.model.embedding.forward(ctx), None
        for i, (run, mem) in enumerate(zip(rep.model.spec.order, rep.runner.memory)):
            layer = rep.model.layers[run.layer]
            hidden, residual = base.BLOCKS[layer.block](layer, hidden, residual, ctx, mem)
            now = ResidualStream(hidden.x.clone(), hidden.a, post=hidden.post).take()[0]
            torch.testing.assert_close(now.cpu().double(), want[i], atol=2e-5, rtol=1e-5, msg=lambda m: f"after layer {i}: {m}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_then_token_by_token(case, dtype):
    """The last tokens one by one: more of them than a page and than most windows hold."""
    name, folder, config, prompts, oracle, rows = case
    rep = replayer(folder, dtype, 256)
    got = {}
    for r, p in enumerate(prompts):
        head = max(0, len(p) - 80)
        if head:
            got[(r, head - 1)] = rep.step([{"id": f"r{r}", "tokens": p[:head], "want": [head - 1]}], [])[0]
        for pos in range(head, len(p)):
            got[(r, pos)] = rep.step([{"id": f"r{r}", "tokens": [p[pos]], "want": [0]}], [f"r{r}"] if pos == len(p) - 1 else [])[0]
    check(got, rows, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_down_to_two_tokens(case, dtype):
    name, folder, config, prompts, oracle, rows = case
    rep = replayer(folder, dtype, 256)
    sizes = [2, 7, 3, 16, 2, 5, 31, 2, 64, 9, 1, 33]
    got = {}
    for r, p in enumerate(prompts):
        pos, i = 0, r
        while pos < len(p):
            n = min(sizes[i % len(sizes)], len(p) - pos)
            i += 1
            want = sorted({0, n - 1})
            logits = rep.step([{"id": f"r{r}", "tokens": p[pos:pos + n], "want": want}], [f"r{r}"] if pos + n == len(p) else [])
            for j, w in enumerate(want):
                got[(r, pos + w)] = logits[j]
            pos += n
    check(got, rows, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_on_pages_and_slots_used_again(case, dtype):
    """Nine unequal requests, at most four live, on a pool that holds the first four: later requests
    start on pages and in state slots that earlier ones have written and given back, beside others
    that are in the middle of theirs. A stale convolution state or a stale page shows in the logits."""
    name, folder, config, _, oracle, _ = case
    lengths = [129, 70, 40, 1, 65, 100, 128, 30, 150]
    prompts = [prompt(900 + i, n, config.vocab) for i, n in enumerate(lengths)]
    rows = [oracle.logits(p) for p in prompts]
    pool = sum(-(-n // 64) for n in lengths[:4])
    rep = replayer(folder, dtype, 64 * pool)
    assert rep.manager.num_blocks == pool and len(rep.manager.free_state_slots) == 4
    chunk = [13, 2, 1, 7, 1, 1, 30, 1, 3, 1]
    cursors, pages = [0] * len(prompts), [-(-n // 64) for n in lengths]
    waiting, live, tick, got, slots_used = list(range(len(prompts))), [], 0, {}, []
    while waiting or live:
        while waiting and len(live) < 4 and sum(pages[r] for r in live) + pages[waiting[0]] <= pool:
            live.append(waiting.pop(0))
        batch, end, wanted = [], [], []
        new = [r for r in live if cursors[r] == 0]
        for r in live:
            n = min(lengths[r] - cursors[r], chunk[(tick + 3 * r) % len(chunk)])
            batch.append({"id": f"q{r}", "tokens": prompts[r][cursors[r]:cursors[r] + n], "want": [n - 1]})
            wanted.append((r, cursors[r] + n - 1))
            cursors[r] += n
            if cursors[r] == lengths[r]:
                end.append(r)
        logits = rep.step(batch, [])
        slots_used += [rep.manager.state_slot(rep.ids[f"q{r}"]) for r in new]
        for j, key in enumerate(wanted):
            got[key] = logits[j]
        rep.step([], [f"q{r}" for r in end])
        live = [r for r in live if r not in end]
        tick += 1
    assert len(slots_used) > len(set(slots_used)), "state slots were used again"
    check(got, rows, dtype)
    assert rep.manager.num_available_blocks() == rep.manager.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_whole_and_in_long_portions(case, dtype):
    """Steps of hundreds of tokens take kernels of their own (heads and values behind the convolution in 16-byte
    pieces and tiles, experts on wide tiles): a prompt of 520 tokens whole, and cut where the second portion
    starts in the middle of a page, beside a short request."""
    name, folder, config, _, oracle, _ = case
    long, short = prompt(321, 520, config.vocab), prompt(322, 40, config.vocab)
    rows = [oracle.logits(long), oracle.logits(short)]
    rep = replayer(folder, dtype, 640)
    marks = [0, 1, 255, 256, 257, 300, 518, 519]
    got = {}
    logits = rep.step([{"id": "w", "tokens": long, "want": marks}], ["w"])
    for j, pos in enumerate(marks):
        got[(0, pos)] = logits[j]
    check(got, rows, dtype)
    got = {}
    logits = rep.step([{"id": "a", "tokens": long[:263], "want": [0, 262]}, {"id": "b", "tokens": short[:7], "want": [6]}], [])
    got[(0, 0)], got[(0, 262)], got[(1, 6)] = logits[0], logits[1], logits[2]
    logits = rep.step([{"id": "b", "tokens": short[7:], "want": [0, 32]}, {"id": "a", "tokens": long[263:], "want": [0, 1, 37, 256]}], ["a", "b"])
    got[(1, 7)], got[(1, 39)] = logits[0], logits[1]
    for j, pos in enumerate([263, 264, 300, 519]):
        got[(0, pos)] = logits[2 + j]
    check(got, rows, dtype)
    assert rep.manager.num_available_blocks() == rep.manager.num_blocks


def test_a_batch_equals_each_request_alone_in_float32(case):
    """float32: the logits of a request do not depend on what else is in the batch, beyond rounding."""
    name, folder, config, prompts, oracle, rows = case
    rep = replayer(folder, "float32", 1024)
    alone = [rep.step([{"id": f"a{r}", "tokens": p, "want": [len(p) - 1]}], [f"a{r}"])[0] for r, p in enumerate(prompts)]
    together = rep.step([{"id": f"b{r}", "tokens": p, "want": [len(p) - 1]} for r, p in enumerate(prompts)],
                        [f"b{r}" for r in range(len(prompts))])
    for r in range(len(prompts)):
        torch.testing.assert_close(together[r], alone[r], atol=2e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(case, dtype):
    """300 tokens fed one by one after a prompt of five: the convolution state is carried through every
    step, windows pass over decoded tokens, the query multiplier steps, the keys fill page after page."""
    name, folder, config, _, oracle, _ = case
    p = prompt(77, 305, config.vocab)
    rows = oracle.logits(p)
    rep = replayer(folder, dtype, 320)
    rep.step([{"id": "d", "tokens": p[:5], "want": []}], [])
    got = {}
    for pos in range(5, len(p)):
        logits = rep.step([{"id": "d", "tokens": [p[pos]], "want": [0]}], [])
        if pos % 7 == 0 or pos >= 300:
            got[(0, pos)] = logits[0]
    check(got, [rows], dtype)


# ---- generation through the engine's entry point -----------------------------------------------------

def test_greedy_generation_through_the_scheduler(case):
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    name, folder, config, prompts, oracle, _ = case
    prompts = [p for p in prompts if len(p) <= 75] + [prompt(42, 90, config.vocab)]
    want = [oracle.greedy(p, 12) for p in prompts]
    sc = SchedulerConfig(max_model_len=256, max_num_seqs=4, max_num_batched_tokens=48, max_prefill_chunk=32)
    llm = LLM(folder, sc, CacheConfig(block_size=32), dtype=torch.float32, num_blocks=24)
    got = llm.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert [r.token_ids[0] for r in got] == want
    # bfloat16 may flip a near-tie: its tokens are judged by the plain model's logits for the same history
    llm16 = LLM(folder, sc, CacheConfig(block_size=32), dtype=torch.bfloat16, num_blocks=24)
    got16 = llm16.generate(prompts[:2], SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True))
    spread = float(oracle.logits(prompts[1]).std())
    for p, r in zip(prompts, got16):
        ids = list(p)
        for tok in r.token_ids[0]:
            row = oracle.logits(ids)[-1]
            assert float(row.max() - row[tok]) <= 0.15 * spread, "a bfloat16 token far from the plain model's best"
            ids.append(tok)


def test_forked_continuations_and_preemption(case):
    """n = 3 at temperature 0: the continuations part after the prompt, each with a copy of the
    convolution state and the prompt's pages shared; all three must be the oracle's greedy continuation.
    And a pool so small that requests are preempted and fed again from their first token."""
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    name, folder, config, prompts, oracle, _ = case
    p = prompt(11, 45, config.vocab)
    want = oracle.greedy(p, 10)
    sc = SchedulerConfig(max_model_len=128, max_num_seqs=4, max_num_batched_tokens=64, max_prefill_chunk=16)
    llm = LLM(folder, sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=24)
    got = llm.generate([p], SamplingParams(max_tokens=10, temperature=0.0, n=3, ignore_eos=True))
    assert got[0].token_ids == [want, want, want]
    many = [prompt(20 + i, 60 + 3 * i, config.vocab) for i in range(4)]
    wants = [oracle.greedy(q, 30) for q in many]
    small = LLM(folder, sc, CacheConfig(block_size=16, caching=False), dtype=torch.float32, num_blocks=14)
    out = small.generate(many, SamplingParams(max_tokens=30, temperature=0.0, ignore_eos=True))
    assert [r.token_ids[0] for r in out] == wants


def test_command_line_generates_from_a_model_folder(case, tmp_path):
    import json
    import os
    import subprocess
    import sys
    name, folder, config, prompts, oracle, _ = case
    if name != "P":
        pytest.skip("one configuration through the command line is enough")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = prompts[2]
    out = tmp_path / "record.json"
    cmd = [sys.executable, "-m", "tinyserve_llm_amd.generate", "--model", folder, "--prompt-ids", ",".join(map(str, p)),
           "--max-tokens", "6", "--temperature", "0", "--ignore-eos", "--dtype", "float32", "--block-size", "32",
           "--num-blocks", "16", "--max-model-len", "256", "--max-num-seqs", "4", "--out", str(out)]
    r = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    record = json.loads(out.read_text())
    text = json.dumps(record)
    assert json.dumps(oracle.greedy(p, 6)).replace(" ", "") in text.replace(" ", ""), text[:500]
