"""The Rugezen decoder on the GPU against the plain implementation in tests/plain/rugezen.py: each
mechanism's kernel alone (with inputs made so that a fault shows: a far key whose score stands out,
keys at page borders and window edges, the first tokens, where the sink weighs most), then whole models
of two small configurations through trace replay (whole, token by token, in portions down to two
tokens, mixed batches on pages and state slots that are used again, long decoding), and greedy
generation through `LLM.generate` and the scheduler. float32 and bfloat16."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import prompt, rugezen_configs
from tests.plain import rugezen as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def hip():
    from tinyserve_llm_amd.ops import hip as h
    return h


def rounded(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """What the kernel gets: rounded to `dtype`; returns (device tensor, the same values in 64-bit on the host)."""
    d = t.to(dtype).to(DEV)
    return d, d.to(F64).cpu()


# ---- the 32-bit stream and the dense feed-forward's pieces ------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [80, 256, 1000])
def test_stream_update_with_two_norms(dtype, width):
    h = hip()
    n = 7
    x = torch.randn(n, width) * 3
    a, a64 = rounded(torch.randn(n, width), dtype)
    b = torch.randn(n, width)                                  # (a branch may also arrive in 32-bit)
    bias, bias64 = rounded(torch.randn(width), dtype)
    w1, w164 = rounded(1 + 0.1 * torch.randn(width), dtype)
    w2, w264 = rounded(1 + 0.1 * torch.randn(width), dtype)
    xd = x.to(DEV)
    h1, h2 = h.stream_update_norm(xd, a, b.to(DEV), bias, 0.37, (w1, w2), 1e-5, out_dtype=dtype)
    want = x.to(F64) + 0.37 * (a64 + b.to(F64) + bias64)
    torch.testing.assert_close(xd.cpu().to(F64), want, atol=2e-6, rtol=1e-6)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(h1.cpu().to(F64), plain.weighted_norm(want, w164, 1e-5), **tol)
    torch.testing.assert_close(h2.cpu().to(F64), plain.weighted_norm(want, w264, 1e-5), **tol)
    # only one branch, no norm; then picked rows, in the order asked for, with nothing updated
    before = xd.clone()
    assert h.stream_update_norm(xd, None, b.to(DEV), None, 2.0) == (None, None)
    torch.testing.assert_close(xd.cpu().to(F64), before.cpu().to(F64) + 2.0 * b.to(F64), atol=2e-6, rtol=1e-6)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    kept = xd.clone()
    picked, _ = h.stream_update_norm(xd, weights=(w1, None), eps=1e-5, rows=rows, out_dtype=dtype)
    assert torch.equal(xd, kept)
    torch.testing.assert_close(picked.cpu().to(F64), plain.weighted_norm(kept.cpu().to(F64)[[5, 0, 5]], w164, 1e-5), **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bias_and_activation(dtype):
    h = hip()
    x = torch.randn(9, 104) * 2
    bias, bias64 = rounded(torch.randn(104), dtype)
    z = x.to(F64) + bias64
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=1e-2, rtol=1e-2)
    for name, fn in (("relu2", plain.squared_relu), ("gelu_tanh", plain.gelu_tanh), ("silu", lambda v: v * torch.sigmoid(v)),
                     ("none", lambda v: v)):
        got = h.bias_activation(x.to(DEV), bias, name, dtype)
        torch.testing.assert_close(got.cpu().to(F64), fn(z), **tol)
    assert float(h.bias_activation(torch.full((1, 3), -2.0, device=DEV), None, "relu2", torch.float32).abs().max()) == 0.0


def test_embedding_into_the_stream():
    h = hip()
    table = torch.randn(50, 72).to(torch.bfloat16).to(DEV)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    out = h.embedding_stream(table, ids)
    assert out.dtype == torch.float32 and torch.equal(out, table[ids.long()].float())


# ---- minGRU ------------------------------------------------------------------------------------

@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [16, 100])
def test_mingru_scan_over_unequal_requests_and_steps(in_dtype, width):
    """Requests of 1, 2, 37, 300 and 700 tokens in one step (the longest is cut into stretches), each
    from a slot that already holds state, then a second step that goes on from what the first left."""
    h = hip()
    lengths = [1, 2, 37, 300, 700]
    slots = [3, 0, 5, 1, 4]
    state0 = torch.rand(6, width)
    bias, bias64 = rounded(torch.randn(2 * width), in_dtype)
    state = state0.to(DEV)
    want_state = state0.to(F64)
    for step in range(2):
        total = sum(lengths)
        zxg, zxg64 = rounded(torch.randn(total, 3 * width) * 2, in_dtype)
        cu = [0]
        for n in lengths:
            cu.append(cu[-1] + n)
        out = h.mingru_scan(zxg, bias, state, torch.tensor(cu, dtype=torch.int32, device=DEV),
                            torch.tensor(slots, dtype=torch.int32, device=DEV), max(lengths), torch.float32)
        for s, slot in enumerate(slots):
            rows = zxg64[cu[s]:cu[s + 1]]
            want, last = plain.mingru_walk(rows[:, :width] + bias64[:width], rows[:, width:2 * width] + bias64[width:],
                                           rows[:, 2 * width:], want_state[slot])
            torch.testing.assert_close(out[cu[s]:cu[s + 1]].cpu().to(F64), want, atol=3e-5, rtol=1e-5)
            want_state[slot] = last
        torch.testing.assert_close(state.cpu().to(F64), want_state, atol=1e-5, rtol=1e-5)
        assert torch.equal(state[2].cpu(), state0[2]), "a slot of no request is left alone"
        lengths = [2, 1, 1, 64, 33]


@pytest.mark.parametrize("n", [100, 127, 128, 129, 1024])
def test_mingru_cuts_equal_the_plain_walk_closely(n):
    """The same portion walked by one wave, cut into stretches for the waves of one workgroup (fewer than
    128 tokens), and cut into chunks of 32 for two kernels (from 128 on): 32-bit rounding apart."""
    h = hip()
    width = 200
    zxg = (torch.randn(n, 3 * width) * 2).to(DEV)
    cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    slot = torch.tensor([1], dtype=torch.int32, device=DEV)
    s1 = torch.rand(2, width, device=DEV)
    s2 = s1.clone()
    # (told 1: a single wave; the kernel walks the whole portion whatever it is told)
    one = h.mingru_scan(zxg, None, s1, cu, slot, 1, torch.float32)
    cut = h.mingru_scan(zxg, None, s2, cu, slot, n, torch.float32)
    assert h.mingru_waves(1) == 1 and h.mingru_waves(127) == 3 and h.MINGRU_CHUNKS_FROM == 128
    torch.testing.assert_close(cut, one, atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(s2, s1, atol=2e-6, rtol=1e-5)
    assert torch.equal(s2[0], s1[0])


# ---- rotation, head norms and the cache write; attention over pages ----------------------------

def paged(pages: int, page: int, G: int, D: int, V: int, dtype):
    """A cache of its own for a kernel test: keys [pages, page, G, D], values kept transposed inside a
    page as the engine's pools keep them."""
    k = torch.zeros(pages, G, page, D, dtype=dtype, device=DEV).permute(0, 2, 1, 3)
    v = torch.zeros(pages, G, V, page, dtype=dtype, device=DEV).permute(0, 3, 1, 2)
    return k, v


SHAPES = [  # heads, kv heads, key size, value size, dims that turn, interleaved, base
    (4, 2, 32, 48, 16, True, 10000.0),
    (2, 2, 16, 16, 16, True, 700.0),
    (6, 1, 24, 8, 4, True, 50000.0),
    (3, 3, 96, 64, 48, False, 500.0),
    (8, 2, 128, 128, 0, True, 1.0),
    (1, 1, 200, 256, 100, True, 1e6),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_rotation_norms_and_cache_write(dtype, shape):
    h = hip()
    H, G, D, V, rot, inter, base = shape
    n, page = 45, 16
    qkv = torch.randn(n, (H + G) * D + G * V) * 1.7
    positions = torch.tensor([0, 1, 2, 3, 100, 1000, 77777] + list(range(5000, 5000 + n - 7)), dtype=torch.int32)
    order = torch.randperm(4 * page)[:n].to(torch.int32)          # any slots, in any order
    order[5] = -1                                                 # an idle row writes nothing
    k, v = paged(4, page, G, D, V, dtype)
    freqs = (base ** (-2.0 * torch.arange(rot // 2, dtype=F64) / max(rot, 1))).to(DEV) if rot else None
    for eps in (1e-5, None):
        k.zero_(); v.zero_()
        q = h.qkv_finish(qkv.to(DEV), freqs, positions.to(DEV), order.to(DEV), k, v, H, G, D, V, dtype, interleaved=inter,
                         qk_norm_eps=eps, v_norm_eps=eps)
        x = qkv.to(F64)
        q64 = plain.turn_pairs(x[:, :H * D].reshape(n, H, D), positions, rot, base, inter)
        k64 = plain.turn_pairs(x[:, H * D:(H + G) * D].reshape(n, G, D), positions, rot, base, inter)
        v64 = x[:, (H + G) * D:].reshape(n, G, V)
        if eps is not None:
            q64, k64, v64 = plain.unit_rms(q64, eps), plain.unit_rms(k64, eps), plain.unit_rms(v64, eps)
        tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=1e-2)
        torch.testing.assert_close(q.cpu().to(F64), q64, **tol)
        kc, vc = k.reshape(4 * page, G, D).cpu().to(F64), v.reshape(4 * page, G, V).cpu().to(F64)
        used = torch.zeros(4 * page, dtype=torch.bool)
        for t in range(n):
            if order[t] >= 0:
                used[order[t]] = True
                torch.testing.assert_close(kc[order[t]], k64[t], **tol)
                torch.testing.assert_close(vc[order[t]], v64[t], **tol)
        assert float(kc[~used].abs().max()) == 0.0 and float(vc[~used].abs().max()) == 0.0


def attention_case(dtype, H, G, D, V, page, length, queries, stand_out, scale, softcap, sink, window=0, seed=0):
    """Keys and values of one request of `length` tokens on shuffled pages, queries at the positions
    `queries`; `stand_out` maps a query's position to the key position whose score is made to stand out
    for it (the key is set to three times the query's direction: a score of 3 sqrt(D) at scale D^-1/2,
    among scores of about 1). Returns (kernel output, oracle output)."""
    h = hip()
    gen = torch.Generator().manual_seed(seed)
    k64 = plain.unit_rms(torch.randn(length, G, D, generator=gen, dtype=F64), 0.0)
    v64 = torch.randn(length, G, V, generator=gen, dtype=F64)
    q64 = plain.unit_rms(torch.randn(len(queries), H, D, generator=gen, dtype=F64), 0.0)
    for i, p in enumerate(queries):
        if p in stand_out:
            # every head of the group looks the same way, and the chosen key lies that way
            g_dir = plain.unit_rms(torch.randn(G, D, generator=gen, dtype=F64), 0.0)
            for hh in range(H):
                q64[i, hh] = g_dir[hh // (H // G)]
            k64[stand_out[p]] = 3 * g_dir
    pages = -(-length // page)
    table = torch.randperm(pages + 3, generator=gen)[:pages].to(torch.int32)
    k, v = paged(pages + 3, page, G, D, V, dtype)
    kr, vr = k64.to(dtype), v64.to(dtype)
    for p in range(length):
        pg = int(table[p // page])
        k[pg, p % page] = kr[p].to(DEV)
        v[pg, p % page] = vr[p].to(DEV)
    q = q64.to(dtype).to(DEV)
    out = h.paged_attention_general(q, k, v, table.view(1, -1).to(DEV), torch.zeros(len(queries), dtype=torch.int32, device=DEV),
                                    torch.tensor(queries, dtype=torch.int32, device=DEV), scale, softcap=softcap, sink=sink,
                                    window=window)
    want = plain.sink_attention(q.cpu().to(F64), kr.to(F64), vr.to(F64), torch.tensor(queries), scale, softcap, sink, window)
    return out.cpu().to(F64), want, vr.to(F64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 32, 48), (2, 2, 16, 16), (6, 1, 24, 8), (6, 2, 96, 96)])
def test_attention_far_keys_page_borders_and_first_tokens(dtype, sizes):
    H, G, D, V = sizes
    page, length = 16, 700
    # a key hundreds of tokens back, keys at both sides of page borders, the query's own key, and the first tokens
    stand_out = {699: 3, 650: 15, 651: 16, 652: 17, 653: 653, 500: 255, 501: 256, 31: 0}
    queries = [0, 1, 2, 3, 15, 16, 17, 31, 500, 501, 650, 651, 652, 653, 699]
    tol = dict(atol=2e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    out, want, v = attention_case(dtype, H, G, D, V, page, length, queries, stand_out, D ** -0.5, 30.0, True)
    torch.testing.assert_close(out, want, **tol)
    # the stand-out key really decides the row: the output is nearly its value
    i = queries.index(699)
    assert float((want[i, 0] - v[3, 0]).abs().max()) < 0.2 * float(v[3, 0].abs().max())
    # without cap and without sink, and with a cap so low that every score is bent
    for cap, sink in ((0.0, False), (0.0, True), (0.7, True), (0.7, False)):
        out, want, _ = attention_case(dtype, H, G, D, V, page, 90, [0, 1, 5, 17, 89], {89: 2}, 0.9 / D ** 0.5, cap, sink, seed=1)
        torch.testing.assert_close(out, want, **tol)


def step_context(table, page, starts, counts):
    """A packed step over requests that all read the pages `table` names: request i feeds `counts[i]`
    tokens from position `starts[i]`."""
    from tinyserve_llm_amd.parts.base import StepContext
    positions, seq_of, cu = [], [], [0]
    for i, (s0, n) in enumerate(zip(starts, counts)):
        positions += list(range(s0, s0 + n))
        seq_of += [i] * n
        cu.append(cu[-1] + n)
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ends = [a + b for a, b in zip(starts, counts)]
    return StepContext(num_tokens=len(positions), num_seqs=len(starts), token_ids=dev([0] * len(positions)), positions=dev(positions),
                       seq_of_token=dev(seq_of), cu_seqlens=dev(cu), context_lens=dev(ends), state_slots=dev([0] * len(starts)),
                       slot_mapping=[], block_tables=[table.view(1, -1).repeat(len(starts), 1).contiguous().to(DEV)],
                       host_cu_seqlens=cu, host_starts=list(starts), host_context_lens=ends, host_state_slots=[0] * len(starts),
                       page_size=page), positions


@pytest.mark.parametrize("sizes", [(6, 3, 96, 96), (8, 2, 64, 64), (2, 2, 128, 128), (4, 4, 32, 32), (16, 1, 64, 64)])
@pytest.mark.parametrize("cap, sink", [(30.0, True), (0.0, True), (0.8, False)])
def test_matrix_core_kernels_general_variants(sizes, cap, sink):
    """bfloat16 heads of the matrix-core kernels' sizes go to those kernels' general variants: single
    tokens (whole walks and walks cut into chunks), a long portion, and single tokens leading a portion
    in one step; far keys, keys at both sides of page borders and of the 32-key steps, the first tokens."""
    h = hip()
    H, G, D, V = sizes
    page, length = 32, 2300
    stand_out = {2299: 3, 2250: 31, 2251: 32, 2252: 33, 2253: 2253, 2200: 63, 2201: 64, 2100: 1023, 2101: 1024, 40: 0, 2222: 2221}
    gen = torch.Generator().manual_seed(5)
    k64 = plain.unit_rms(torch.randn(length, G, D, generator=gen, dtype=F64), 0.0)
    v64 = torch.randn(length, G, V, generator=gen, dtype=F64)
    q64 = plain.unit_rms(torch.randn(length, H, D, generator=gen, dtype=F64), 0.0)
    for p, key in stand_out.items():
        g_dir = plain.unit_rms(torch.randn(G, D, generator=gen, dtype=F64), 0.0)
        for hh in range(H):
            q64[p, hh] = g_dir[hh // (H // G)]
        k64[key] = 3 * g_dir
    pages = -(-length // page)
    table = torch.randperm(pages + 5, generator=gen)[:pages].to(torch.int32)
    k, v = paged(pages + 5, page, G, D, V, torch.bfloat16)
    kr, vr = k64.to(torch.bfloat16), v64.to(torch.bfloat16)
    idx = (table.long()[torch.arange(length) // page], torch.arange(length) % page)
    k[idx[0].to(DEV), idx[1].to(DEV)] = kr.to(DEV)
    v[idx[0].to(DEV), idx[1].to(DEV)] = vr.to(DEV)
    qr = q64.to(torch.bfloat16)
    scale = D ** -0.5
    tol = dict(atol=2e-2, rtol=2e-2)

    def run(starts, counts):
        ctx, positions = step_context(table, page, starts, counts)
        q = qr[positions].to(DEV).contiguous()
        assert h.decode_kernel_takes(q, k, v), "these sizes are the matrix-core kernels'"
        out = h.paged_attention(q, k, v, ctx, 0, scale, 0, softcap=cap, sink=sink)
        want = plain.sink_attention(qr[positions].to(F64), kr.to(F64), vr.to(F64), torch.tensor(positions), scale, cap, sink)
        torch.testing.assert_close(out.cpu().to(F64), want, msg=lambda m: f"starts {starts} counts {counts}: {m}", **tol)

    for pos in (0, 1, 31, 32, 40, 2100, 2101, 2299):
        run([pos], [1])                                   # one token, one request
    run([2299, 40, 2250, 0, 2201, 2222, 33, 2100], [1] * 8)   # a batch of single tokens of unequal contexts
    run([2180], [120])                                    # a portion deep in a request
    run([0], [70])                                        # the first tokens as a portion
    run([2252, 2253, 2190], [1, 1, 110])                  # single tokens lead a portion
    run([2296], [2])                                      # a portion of two tokens


def test_the_sink_weighs_most_on_the_first_tokens():
    """One visible key of score s: the weight is e^s / (1 + e^s), not 1."""
    out, want, v = attention_case(torch.float32, 2, 1, 16, 16, 16, 3, [0], {}, 0.25, 40.0, True)
    torch.testing.assert_close(out, want, atol=1e-6, rtol=1e-5)
    assert float((out[0, 0] / v[0, 0]).mean()) < 0.9
    no_sink, _, _ = attention_case(torch.float32, 2, 1, 16, 16, 16, 3, [0], {}, 0.25, 40.0, False)
    torch.testing.assert_close(no_sink[0, 0], v[0, 0], atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_window_edges(dtype):
    """The kernel's window: the key just inside decides the row, the key just outside is not seen."""
    H, G, D, V, window = 2, 1, 32, 16, 40
    tol = dict(atol=2e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    inside = {200: 200 - window + 1, 201: 201 - window + 1}
    out, want, v = attention_case(dtype, H, G, D, V, 16, 260, [200, 201, 259], inside, D ** -0.5, 0.0, True, window)
    torch.testing.assert_close(out, want, **tol)
    assert float((want[0, 0] - v[161, 0]).abs().max()) < 0.2 * float(v[161, 0].abs().max())
    outside = {200: 200 - window, 259: 259 - window}
    out, want, v = attention_case(dtype, H, G, D, V, 16, 260, [200, 201, 259], outside, D ** -0.5, 0.0, True, window)
    torch.testing.assert_close(out, want, **tol)
    assert float((want[0, 0] - v[160, 0]).abs().max()) > 0.5


# ---- whole models through trace replay ---------------------------------------------------------

LENGTHS = {"P": [1, 2, 40, 150], "Q": [3, 66, 129, 200], "R": [1, 7, 65, 140], "S": [2, 33, 64, 130]}
# Bounds on a logit's error as a share of the logits' spread (their standard deviation over the oracle's rows).
# float32: only the engine's own 32-bit rounding separates it from the 64-bit oracle (worst seen 4e-6 of the spread).
# bfloat16: activations are rounded to 8 bits of mantissa at every projection's input; the worst logit was off by
# 1.2 to 2.6 % of the spread, configuration by configuration, in every way of feeding; the bound is twice the largest.
TOL = {"float32": 2e-5, "bfloat16": 5e-2}


@pytest.fixture(scope="module", params=["P", "Q", "R", "S"])
def case(request, tmp_path_factory):
    from tinyserve_llm_amd.weights.random_init import write_random_model
    name = request.param
    config, seed = rugezen_configs()[name]
    folder = str(tmp_path_factory.mktemp(f"rugezen_{name}"))
    write_random_model(folder, config, seed, torch.bfloat16)
    oracle = plain.PlainRugezen(folder)
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
        # the residual stream after every layer run, layer by layer
        from tinyserve_llm_amd.engine.runner import StepEntry
        from tinyserve_llm_amd.parts import base
        from tinyserve_llm_amd.parts.stream import ResidualStream
        p = prompts[2]
        want = oracle.streams(p)
        rep.manager.allocate(77, p)
        ctx, _, _ = rep.runner.prepare([StepEntry(77, p, 0, [])])
        ctx.position_encodings = rep.model.position_encodings
        hidden, residual = rep.model.embedding.forward(ctx), None
        for i, (run, mem) in enumerate(zip(rep.model.spec.order, rep.runner.memory)):
            layer = rep.model.layers[run.layer]
            hidden, residual = base.BLOCKS[layer.block](layer, hidden, residual, ctx, mem)
            now = ResidualStream(hidden.x.clone(), hidden.a, hidden.b, hidden.bias, hidden.mult).settle()[0]
            torch.testing.assert_close(now.cpu().double(), want[i], atol=2e-5, rtol=1e-5, msg=lambda m: f"after run {i}: {m}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_then_token_by_token(case, dtype):
    """The last tokens one by one: more of them than a page holds, so decoding crosses page borders."""
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
    that are in the middle of theirs. Stale state or a stale page shows in the logits."""
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
    """300 tokens fed one by one after a prompt of five: the state is carried through every step and
    the keys fill page after page."""
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


# ---- generation through the engine's entry point -----------------------------------------------

def test_greedy_generation_through_the_scheduler(case):
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    name, folder, config, prompts, oracle, _ = case
    prompts = [p for p in prompts if len(p) <= 70] + [prompt(42, 90, config.vocab)]
    want = [oracle.greedy(p, 12) for p in prompts]
    sc = SchedulerConfig(max_model_len=256, max_num_seqs=4, max_num_batched_tokens=48, max_prefill_chunk=32)
    llm = LLM(folder, sc, CacheConfig(block_size=32), dtype=torch.float32, num_blocks=24)
    got = llm.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert [r.token_ids[0] for r in got] == want
    # bfloat16 may flip a near-tie: its tokens are judged by the plain model's logits for the same history
    llm16 = LLM(folder, sc, CacheConfig(block_size=32), dtype=torch.bfloat16, num_blocks=24)
    got16 = llm16.generate(prompts[:2], SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True))
    for p, r in zip(prompts, got16):
        ids = list(p)
        for tok in r.token_ids[0]:
            row = oracle.logits(ids)[-1]
            assert float(row.max() - row[tok]) <= 0.1, "a bfloat16 token far from the plain model's best"
            ids.append(tok)


def test_forked_continuations_copy_state_and_pages(case):
    """n = 3 at temperature 0: the continuations part after the prompt, each with a copy of the minGRU
    state and the prompt's pages shared; all three must be the oracle's greedy continuation. And a pool
    so small that requests are preempted and fed again from their first token (their state slot
    starts from zero again)."""
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
    # four requests of 60 to 70 tokens that grow by 30 on 14 pages of 16: they do not all fit to the end
    many = [prompt(20 + i, 60 + 3 * i, config.vocab) for i in range(4)]
    wants = [oracle.greedy(q, 30) for q in many]
    small = LLM(folder, sc, CacheConfig(block_size=16, caching=False), dtype=torch.float32, num_blocks=14)
    out = small.generate(many, SamplingParams(max_tokens=30, temperature=0.0, ignore_eos=True))
    assert [r.token_ids[0] for r in out] == wants
    assert small.scheduler.stats().preemptions > 0, "the pool was meant to be too small"


def test_command_line_generates_from_a_model_folder(case, tmp_path):
    import json
    import os
    import subprocess
    import sys
    name, folder, config, prompts, oracle, _ = case
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


@pytest.mark.parametrize("rows", [1, 3, 8])
@pytest.mark.parametrize("activation", ["relu2", "gelu_tanh", "silu"])
def test_projection_with_bias_and_activation_on_the_way_out(rows, activation):
    """Few rows: the up projection's kernel applies bias and activation to its 32-bit sums itself."""
    h = hip()
    K, N = 512, 328
    x, x64 = rounded(torch.randn(rows, K), torch.bfloat16)
    w, w64 = rounded(torch.randn(N, K) * 0.05, torch.bfloat16)
    b, b64 = rounded(torch.randn(N), torch.bfloat16)
    assert h.skinny8_act_takes(x, w, b)
    fn = {"relu2": plain.squared_relu, "gelu_tanh": plain.gelu_tanh, "silu": lambda v: v * torch.sigmoid(v)}[activation]
    want = fn(x64 @ w64.T + b64)
    got32 = h.gemm_skinny8_act(x, w, b, activation, torch.float32)
    torch.testing.assert_close(got32.cpu().to(F64), want, atol=2e-5, rtol=2e-5)
    got16 = h.gemm_skinny8_act(x, w, b, activation, torch.bfloat16, h.pack_weight8(w))
    torch.testing.assert_close(got16.cpu().to(F64), want, atol=2e-2, rtol=1e-2)
    none = h.gemm_skinny8_act(x, w, None, activation, torch.float32)
    torch.testing.assert_close(none.cpu().to(F64), fn(x64 @ w64.T), atol=2e-5, rtol=2e-5)
