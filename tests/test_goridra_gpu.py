"""Goridra in the engine against its plain implementation (tests/plain_goridra.py): each mechanism alone at the
kernels, then whole models in every way of cutting the work.

In bf16 a router's near tie may fall the other way than in float64, which changes a token's output by far more than
rounding. The model tests in bf16 therefore hand the plain implementation the experts that the engine chose, and
check separately that the engine's choice is the plain one wherever the scores are not close.
"""
import math

import numpy as np
import pytest
import torch

import goridra_helpers as gh
import helpers
import plain_goridra as pg
from test_kernels_gpu import FakeStep, dev, ints, paged_setup, rounded

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
# Largest |logit difference| from the float64 plain implementation, as a fraction of the request's largest |logit|.
# fp32: the rounding of a few thousand fused multiply-adds a value over five layers (measured: up to 5.5e-6 at 457
# tokens; a key too many or too few, a wrong expert or a lost page shows as 1e-2 and more). bf16: activations and cache
# rounded to 8 bits of mantissa at every part.
TOL = {"float32": 1e-5, "bfloat16": 2.5e-2}


# ---- mechanisms alone ----------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [5, 48, 256, 1000, 4096])
def test_layernorm(ops32, dtype, width):
    rng = np.random.default_rng(width)
    x = (rng.standard_normal((9, width)) * 3 + 50.0 * rng.standard_normal((9, 1))).astype(np.float32)   # rows far from zero
    w, b = rng.standard_normal(width).astype(np.float32), rng.standard_normal(width).astype(np.float32)
    out = torch.empty((9, width), dtype=dtype, device="cuda")
    ops32.layernorm(dev(x), dev(w), dev(b), 1e-5, out)
    want = pg.layer_norm(x.astype(np.float64), w, b, 1e-5)
    tol = 3e-5 if dtype == torch.float32 else 0.03
    assert np.max(np.abs(out.float().cpu().numpy() - want)) <= tol * max(1.0, np.max(np.abs(want)) / 4)
    rows = [7, 0, 7, 3]
    some = torch.empty((4, width), dtype=dtype, device="cuda")
    ops32.layernorm(dev(x), dev(w), None, 1e-5, some, rows=ints(rows))
    want = pg.layer_norm(x.astype(np.float64), w, 0.0, 1e-5)[rows]
    assert np.max(np.abs(some.float().cpu().numpy() - want)) <= tol * max(1.0, np.max(np.abs(want)) / 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_activations_and_soft_cap(ops32, dtype):
    rng = np.random.default_rng(1)
    z = rounded((rng.standard_normal((7, 130)) * 3).astype(np.float32), dtype)
    want = {"gelu_erf": pg.gelu_erf(z.astype(np.float64)), "relu2": np.maximum(z.astype(np.float64), 0.0) ** 2,
            "gelu_tanh": 0.5 * z * (1 + np.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z.astype(np.float64) ** 3)))}
    for kind, w in want.items():
        out = torch.empty((7, 130), dtype=dtype, device="cuda")
        ops32.activation(kind, dev(z, dtype), out)
        tol = 2e-6 if dtype == torch.float32 else 0.008
        assert np.max(np.abs(out.float().cpu().numpy() - w) / (1 + np.abs(w))) <= tol, kind
    x = dev((rng.standard_normal((5, 77)) * 40).astype(np.float32))
    want = 11.0 * np.tanh(x.cpu().numpy().astype(np.float64) / 11.0)
    ops32.softcap(x, 11.0)
    assert np.max(np.abs(x.cpu().numpy() - want)) <= 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (8, 384, 256), (16, 4608, 3584), (20, 1000, 1024), (33, 200, 1000), (100, 256, 512),
                                   (128, 1024, 2048), (300, 512, 256), (2048, 1024, 512), (700, 8192, 2048), (5, 100, 33)])
def test_product_with_an_activation_in_its_last_lines(ops32, ops16, dtype, M, N, K):
    """``gemm(..., activation=)`` at shapes that go to every product kernel (few rows that finish their outputs, K cut
    over waves and blocks, tiles through LDS, the plain kernel), with a bias, against the plain product and function."""
    ops = ops32 if dtype == torch.float32 else ops16
    rng = np.random.default_rng(M + N + K)
    a = rounded(rng.standard_normal((M, K)).astype(np.float32), dtype)
    w = rounded((rng.standard_normal((N, K)) / math.sqrt(K) * 2).astype(np.float32), dtype)
    bias = rng.standard_normal(N).astype(np.float32)
    z = a @ w.T + bias
    for kind, want in (("gelu_erf", pg.gelu_erf(z)), ("relu2", np.maximum(z, 0.0) ** 2)):
        out = torch.empty((M, N), dtype=dtype, device="cuda")
        ops.gemm(dev(a, dtype), dev(w, dtype), out, bias=dev(bias), activation=kind)
        err = np.max(np.abs(out.float().cpu().numpy() - want) / (1 + np.abs(want)))
        assert err <= (2e-5 if dtype == torch.float32 else 0.01), f"{kind}: {err:.3e}"


@pytest.mark.parametrize("E,top,groups,keep", [(10, 3, 2, 1), (6, 2, 3, 2), (5, 1, 1, 1), (4, 4, 4, 4), (16, 3, 4, 2),
                                               (64, 6, 8, 3), (128, 8, 1, 1), (7, 7, 1, 1), (12, 1, 12, 1), (256, 8, 8, 4)])
def test_router(ops32, E, top, groups, keep):
    """Choices and weights against the plain router; logits spread so that no two scores are close, except that a
    few rows hold equal logits on purpose (the lower index wins)."""
    rng = np.random.default_rng(E * 100 + top)
    z = (rng.permuted(np.tile(np.linspace(-4, 4, E), (50, 1)), axis=1) + 0.01 * rng.standard_normal((50, E))).astype(np.float32)
    ids, wts = ops32.moe_route(dev(z), top, groups, keep)
    want_ids, want_w = pg.route(z.astype(np.float64), top, groups, keep)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.max(np.abs(wts.cpu().numpy() - want_w)) <= 2e-6
    assert np.allclose(wts.cpu().numpy().sum(axis=1), 1.0, atol=1e-5)
    ties = np.zeros((3, E), np.float32)
    ids, _ = ops32.moe_route(dev(ties), top, groups, keep)
    assert np.array_equal(ids.cpu().numpy(), pg.route(ties.astype(np.float64), top, groups, keep)[0])


def test_router_drops_the_experts_of_groups_that_lose(ops32):
    """The best single expert sits in a group whose rival holds the next two: with one group kept and three choices
    the lone best still decides the group."""
    z = np.array([[5.0, -9.0, -9.0, -9.0, -9.0, 4.0, 4.1, 3.9, -9.0, -9.0]], np.float32)
    ids, wts = ops32.moe_route(dev(z), 3, 2, 1)
    assert ids.cpu().numpy().tolist() == [[0, 1, 2]]
    ids, _ = ops32.moe_route(dev(z), 3, 2, 2)
    assert ids.cpu().numpy().tolist() == [[0, 6, 5]]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,F,E,top", [(1, 48, 40, 6, 2), (7, 256, 128, 8, 1), (300, 256, 64, 4, 4), (33, 128, 32, 16, 3),
                                         (700, 256, 128, 8, 2), (5, 100, 24, 5, 1), (64, 512, 256, 32, 4), (100, 256, 128, 4, 2),
                                         (900, 384, 96, 3, 1)])
def test_experts(ops32, ops16, dtype, T, W, F, E, top):
    """The experts' weighted sum for given choices, through the plan and the grouped products, against a loop."""
    ops = ops32 if dtype == torch.float32 else ops16
    rng = np.random.default_rng(T + W + E)
    h = rounded(rng.standard_normal((T, W)).astype(np.float32), dtype)
    up = rounded((rng.standard_normal((E, F, W)) / math.sqrt(W)).astype(np.float32), dtype)
    down = rounded((rng.standard_normal((E, W, F)) / math.sqrt(F)).astype(np.float32), dtype)
    ids = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    ids[0] = np.arange(top)                                   # and one expert that may get no row at all
    wts = rng.random((T, top)).astype(np.float32)
    x0 = rng.standard_normal((T, W)).astype(np.float32)
    want = x0.astype(np.float64)
    for t in range(T):
        for e, wt in zip(ids[t], wts[t]):
            a = np.maximum(h[t].astype(np.float64) @ up[e].T, 0.0) ** 2
            if dtype == torch.bfloat16:
                a = helpers.bf16_round(a).astype(np.float64)
            want[t] += wt * (a @ down[e].T)
    for plain in ([False] if dtype == torch.float32 else [False, True]):
        x = dev(x0)
        ops.force_plain_gemm = plain
        try:
            ops.moe_experts(dev(h, dtype), ints(ids).view(T, top), dev(wts), dev(up, dtype), dev(down, dtype), "relu2", x)
        finally:
            ops.force_plain_gemm = False
        err = np.max(np.abs(x.cpu().numpy() - want)) / np.max(np.abs(want))
        assert err <= (1e-5 if dtype == torch.float32 else 1e-2), f"plain={plain}: {err:.3e}"


def chunk_attention(q, k, v, scale, size):
    """Queries at the last len(q) positions of a sequence of len(k) keys, masked by chunks (float64)."""
    n, ql = k.shape[0], q.shape[0]
    full = np.zeros((n,) + q.shape[1:])
    full[n - ql:] = q
    return pg.attend(full, k.astype(np.float64), v.astype(np.float64), scale, size).reshape(n, q.shape[1], -1)[n - ql:]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,page,size,lengths,q_lens", [
    (4, 2, 16, 8, 24, [1, 5, 24, 25, 130, 203], [1, 3, 24, 2, 1, 60]),           # plain kernels: a head of 16
    (6, 1, 8, 8, 7, [50, 63], [50, 1]),                                          # a chunk that no page size divides
    (8, 2, 64, 16, 48, [700, 96, 97, 333, 64], [100, 96, 1, 17, 1]),             # matrix cores: portions beside decoded tokens
    (8, 4, 32, 16, 32, [2100, 1500, 64, 65], [1, 1, 1, 1]),                      # decoded tokens far into long sequences
    (28, 4, 128, 16, 1024, [2100, 1025, 1024], [1, 1, 1]),                       # long chunks: the keys are cut over waves
    (4, 1, 64, 64, 80, [600], [600]),                                            # one prompt, whole; pages larger than a key block
    (2, 2, 128, 16, 200, [1100], [300]),                                         # a portion late in a prompt
    (8, 2, 128, 16, 512, [1500], [1500]),                                        # few blocks, long chunks: a tile's keys cut over blocks
    (8, 2, 64, 16, 700, [2000, 90], [400, 90]),                                  # the same for a portion that starts inside a chunk
    (16, 2, 128, 32, 300, [1203, 2900, 301, 300, 599], [1, 1, 1, 1, 1]),         # decoded tokens at the first, second and last place of a chunk
    (4, 4, 32, 8, 1000, [999, 1000, 1001, 2001], [40, 40, 40, 40]),              # portions across a chunk's border
])
def test_attention_masked_by_chunks(ops32, ops16, dtype, H, G, D, page, size, lengths, q_lens):
    ops = ops32 if dtype == torch.float32 else ops16
    rng = np.random.default_rng(H + D + size)
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, dtype)
    qs, positions, slots, wants = [], [], [], []
    scale = 1.0 / math.sqrt(D)
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q = rng.standard_normal((ql, H, D)).astype(np.float32)
        wants.append(chunk_attention(rounded(q, dtype), rounded(ks[s], dtype), rounded(vs[s], dtype), scale, size))
        qs.append(q)
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * D)
    out = torch.empty((q.shape[0], H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops.paged_attention(dev(q, dtype), H, G, D, cache, step, 0, scale, out, mask_chunk=size)
    err = np.max(np.abs(out.float().cpu().numpy() - want))
    assert err <= (2e-5 if dtype == torch.float32 else 0.02), f"max |diff| {err:.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,page,size,n,ql", [(4, 2, 16, 8, 24, 100, 1), (4, 2, 16, 8, 24, 100, 30), (8, 2, 64, 16, 48, 500, 1),
                                                  (8, 2, 64, 16, 48, 500, 120), (4, 4, 32, 16, 256, 1500, 1), (4, 4, 32, 16, 256, 1500, 300)])
def test_a_key_at_the_edge_of_a_chunk_is_seen_or_not(ops32, ops16, dtype, H, G, D, page, size, n, ql):
    """One key matches every query far better than all others and carries a value of its own. At the first position
    of the last query's chunk it takes the whole output of the queries of that chunk; one position earlier it is
    outside and changes nothing, however well it matches. In a prompt portion and in a decoded token."""
    ops = ops32 if dtype == torch.float32 else ops16
    scale = 1.0 / math.sqrt(D)
    first = (n - 1) // size * size                             # where the last query's chunk starts
    for spike, seen in ((first, True), (first - 1, False), (0, first == 0)):
        rng = np.random.default_rng(n + ql)
        ks, vs, cache, table = paged_setup(rng, [n], G, D, page, torch.float32)
        k, v = ks[0] * 0.1, vs[0]
        direction = np.ones(D, np.float32) / math.sqrt(D)
        k[spike] = 60.0 * direction
        v[spike] = 7.0
        q = (0.1 * rng.standard_normal((ql, H, D)) + 4.0 * direction).astype(np.float32)
        # the same sequence again, in a cache of the kernel's dtype
        kc = np.zeros((cache.k.shape[0], G * D), np.float32)
        vc = np.zeros_like(kc)
        tb = table.cpu().numpy()[0]
        for j in range(n):
            row = tb[j // page] * page + j % page
            kc[row], vc[row] = k[j].reshape(-1), v[j].reshape(-1)
        from test_kernels_gpu import to_value_layout
        cache.k, cache.v = dev(kc, dtype), dev(to_value_layout(vc, page), dtype)
        out = torch.empty((ql, H * D), dtype=dtype, device="cuda")
        step = FakeStep(ints(list(range(n - ql, n))), ints([0] * ql), table, None)
        ops.paged_attention(dev(q.reshape(ql, -1), dtype), H, G, D, cache, step, 0, scale, out, mask_chunk=size)
        got = out.float().cpu().numpy().reshape(ql, H, D)
        want = chunk_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale, size)
        assert np.max(np.abs(got - want)) <= (2e-5 if dtype == torch.float32 else 0.03)
        in_chunk = np.arange(n - ql, n) >= first
        if seen:
            assert np.all(np.abs(got[in_chunk] - 7.0) < 0.1), f"the key at {spike} should take the output"
        else:
            assert np.all(np.abs(got[in_chunk]) < 4.0), f"the key at {spike} should not be seen"


@pytest.mark.parametrize("dtype", DTYPES)
def test_value_heads_of_another_size_masked_by_chunks(ops32, ops16, dtype):
    ops = ops32 if dtype == torch.float32 else ops16
    H, G, D, Dv, page, size, n, ql = 4, 2, 12, 20, 8, 24, 90, 40
    rng = np.random.default_rng(5)
    k = rounded(rng.standard_normal((n, G, D)).astype(np.float32), dtype)
    v = rounded(rng.standard_normal((n, G, Dv)).astype(np.float32), dtype)
    q = rounded(rng.standard_normal((ql, H, D)).astype(np.float32), dtype)
    blocks = -(-n // page)
    perm = rng.permutation(blocks + 2)
    table = np.zeros((1, blocks + 1), np.int32)
    table[0, :blocks] = perm[:blocks]
    kc = np.zeros(((blocks + 2) * page, G * D), np.float32)
    vc = np.zeros(((blocks + 2) * page, G * Dv), np.float32)
    for j in range(n):
        row = table[0, j // page] * page + j % page
        kc[row], vc[row] = k[j].reshape(-1), v[j].reshape(-1)
    from test_kernels_gpu import FakeCache, to_value_layout
    cache = FakeCache(group=0, k=dev(kc, dtype), v=dev(to_value_layout(vc, page), dtype), page_tokens=page, window=0)
    out = torch.empty((ql, H * Dv), dtype=dtype, device="cuda")
    step = FakeStep(ints(list(range(n - ql, n))), ints([0] * ql), ints(table), None)
    ops.paged_attention(dev(q.reshape(ql, -1), dtype), H, G, D, cache, step, 0, 0.3, out, v_head_dim=Dv, mask_chunk=size)
    want = chunk_attention(q, k, v, 0.3, size).reshape(ql, -1)
    assert np.max(np.abs(out.float().cpu().numpy() - want)) <= (2e-5 if dtype == torch.float32 else 0.02)


# ---- whole models ---------------------------------------------------------------------------------------------------

LENGTHS = {"small": [1, 7, 23, 24, 25, 57, 130], "cores": [3, 48, 49, 97, 161, 230]}


@pytest.fixture(scope="module", params=["small", "cores"])
def tiny(request, tmp_path_factory):
    name = request.param
    cfg = gh.CONFIGS[name]
    d = gh.make_model_dir(str(tmp_path_factory.mktemp("goridra_" + name)), cfg, seed=len(name), stored=gh.STORED[name])
    reqs = gh.random_requests(cfg, LENGTHS[name], seed=7)
    return name, cfg, d, reqs, gh.plain_logits(d, reqs)


def engine_for(model_dir, dtype, name, max_tokens, max_seqs=4, graphs=True):
    import hf_cpu_amd
    return hf_cpu_amd.load_engine(model_dir, dtype=dtype, page_tokens=gh.PAGE[name], max_tokens=max_tokens,
                                  max_seqs=max_seqs, graphs=graphs)


def run_against_plain(name, d, reqs, want, dtype, steps, what, graphs=True):
    """Runs the trace; in bf16 with the engine's choice of experts handed to the plain implementation, after checking
    that the choice is the plain one wherever the plain scores are 0.02 or more apart."""
    engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps), graphs=graphs and dtype == "float32")
    if dtype == "float32":
        got = helpers.run_trace_in_engine(engine, steps)
    else:
        with gh.record_choices(engine) as rec:
            got = helpers.run_trace_in_engine(engine, steps)
        cfg, w = pg.read_model(d)
        want = {}
        for r, toks in reqs.items():
            margins, mine = {}, rec.chosen.get(r, {})
            want[r] = gh.forward_with_choices(cfg, w, toks, mine, margins)
            assert set(mine) == set(margins), f"{what}: request {r}: the router did not run once for every token and layer"
            clear = [key for key, (gap, _) in margins.items() if gap >= 0.02]
            assert len(clear) >= len(margins) // 2
            wrong = [key for key in clear if not margins[key][1]]
            assert not wrong, f"{what}: request {r}: at (layer, position) {wrong[:5]} the engine chose other experts than the " \
                              "plain router although the scores are apart"
    worst = helpers.compare(got, want, TOL[dtype], what)
    engine.manager.check()
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)
    return engine, got, worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cutting", ["whole", "tail", "portions", "mixed"])
def test_cuttings(gpu, tiny, dtype, cutting):
    """Whole prompts; most of a prompt and then token by token over several chunk borders; portions of changing size
    down to two tokens; up to four requests live, portions beside single tokens, pages and slots used again."""
    name, cfg, d, reqs, want = tiny
    steps = {"whole": helpers.trace_whole, "tail": lambda r: helpers.trace_tail(r, tail=90),
             "portions": helpers.trace_portions, "mixed": lambda r: helpers.trace_mixed(r, seed=3)}[cutting](reqs)
    engine, got, worst = run_against_plain(name, d, reqs, want, dtype, steps, f"{name} {dtype} {cutting}")
    assert len(got) == sum(len(t) for t in reqs.values())
    print(f"{name} {dtype} {cutting}: worst |diff| {worst:.3e}")
    if cutting == "mixed":
        assert any(p.reused > 0 for p in engine.manager.pools), "the trace was meant to use pages again"


def test_cuttings_agree_with_each_other(gpu, tiny):
    """In fp32 the cuttings agree among themselves far more closely than rounding in bf16 would allow: the same
    values are computed, only in other launches; decoding replays captured graphs."""
    name, cfg, d, reqs, _ = tiny
    results = []
    for make in (helpers.trace_whole, helpers.trace_portions, lambda r: helpers.trace_tail(r, tail=60),
                 lambda r: helpers.trace_mixed(r, seed=5)):
        steps = make(reqs)
        engine = engine_for(d, "float32", name, helpers.max_live_tokens(steps))
        results.append(helpers.run_trace_in_engine(engine, steps))
    for other in results[1:]:
        for key, row in results[0].items():
            err = float(np.max(np.abs(row - other[key])))
            assert err <= 3e-5, f"{name}: {key}: cuttings differ by {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_same_trace_twice_gives_the_same_bits(gpu, tiny, dtype):
    """Where a (token, choice) pair lands inside its expert's run of rows is left to atomics; the values are not: a
    mixed trace replayed in a second engine gives the same logits bit for bit."""
    name, cfg, d, reqs, _ = tiny
    steps = helpers.trace_mixed(reqs, seed=11)
    runs = []
    for _ in range(2):
        engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps))
        runs.append(helpers.run_trace_in_engine(engine, steps))
    assert runs[0].keys() == runs[1].keys()
    for key, row in runs[0].items():
        assert np.array_equal(row, runs[1][key]), f"{name} {dtype}: {key} differs between two runs"


def test_a_batch_of_unequal_requests_against_each_alone(gpu, tiny):
    name, cfg, d, reqs, want = tiny
    engine = engine_for(d, "float32", name, 64 * len(reqs) + sum(len(t) for t in reqs.values()), max_seqs=len(reqs))
    together = engine.step([(r, toks, list(range(len(toks)))) for r, toks in reqs.items()]).cpu().numpy()
    at = 0
    for r, toks in reqs.items():
        engine.release(r)
        alone = engine.step([(r + "'", toks, list(range(len(toks))))]).cpu().numpy()
        engine.release(r + "'")
        assert np.max(np.abs(alone - together[at:at + len(toks)])) <= 2e-5
        assert np.max(np.abs(alone - want[r])) <= TOL["float32"] * np.max(np.abs(want[r]))
        at += len(toks)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_small_pool(gpu, tiny, dtype):
    """Three requests decoded token by token together from their second token on, in a pool that holds them and no
    more, then three more in the pages and slots that they gave back."""
    name, cfg, d, reqs, want = tiny
    long = {r: t for r, t in reqs.items() if len(t) >= 57}
    names = list(long)[:3]
    steps = []
    for turn in range(2):
        ids = {r: f"{r}/{turn}" for r in names}
        steps.append(helpers._step(len(steps), [(ids[r], long[r][:2], [0, 1]) for r in names]))
        for i in range(2, max(len(long[r]) for r in names)):
            live = [r for r in names if i < len(long[r])]
            steps.append(helpers._step(len(steps), [(ids[r], long[r][i:i + 1], [0]) for r in live],
                                       [ids[r] for r in live if i == len(long[r]) - 1]))
    reqs2 = {f"{r}/{turn}": long[r] for r in names for turn in range(2)}
    want2 = {f"{r}/{turn}": want[r] for r in names for turn in range(2)}
    engine, got, _ = run_against_plain(name, d, reqs2, want2, dtype, steps, f"{name} {dtype} long decoding")
    assert all(p.reused > 0 for p in engine.manager.pools)
    if dtype == "float32":
        assert engine.graph_replays > 0, "decode steps were meant to replay captured graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_request_in_a_pool_that_holds_a_chunk_of_it(gpu, tiny, dtype):
    """Pages that lie before every user's current chunk go back while the request runs: its longest request passes
    through a pool far smaller than itself, in portions and then token by token, with the plain logits."""
    name, cfg, d, _, _ = tiny
    largest = max(l["mixer"]["mask"]["size"] for l in cfg["layers"])
    r = "long"
    toks = [int(t) for t in np.random.default_rng(9).integers(0, cfg["vocab"], 2 * largest + 57)]
    want = gh.plain_logits(d, {r: toks}) if dtype == "float32" else None
    steps, at, sizes = [], 0, [9, 2, 7, 1, 8, 3]
    while at < len(toks):
        n = min(sizes[len(steps) % len(sizes)] if at < len(toks) - 40 else 1, len(toks) - at)
        steps.append(helpers._step(len(steps), [(r, toks[at:at + n], range(n))], [r] if at + n == len(toks) else []))
        at += n
    pool = largest + 9 + 2 * gh.PAGE[name]
    assert pool < len(toks) - 30
    import hf_cpu_amd
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=gh.PAGE[name], max_tokens=pool, max_seqs=1,
                                    max_context=len(toks), graphs=dtype == "float32")
    if dtype == "float32":
        got = helpers.run_trace_in_engine(engine, steps)
        helpers.compare(got, {r: want[r]}, TOL[dtype], f"{name} {dtype} small pool")
    else:
        with gh.record_choices(engine) as rec:
            got = helpers.run_trace_in_engine(engine, steps)
        pcfg, w = pg.read_model(d)
        helpers.compare(got, {r: gh.forward_with_choices(pcfg, w, toks, rec.chosen[r])}, TOL[dtype], f"{name} {dtype} small pool")
    engine.manager.check()
    assert all(p.reused > 0 and p.n_held == 0 for p in engine.manager.pools)


def test_trace_replay_program(gpu, tiny, tmp_path):
    """bin/trace_run as a user calls it (pages of 16, four slots, a pool for the live requests only): a mixed trace in
    fp32 against the plain implementation; in bf16 the same trace, where all rows but a router's near ties agree with it."""
    import json
    import os
    import subprocess
    import sys
    name, cfg, d, reqs, want = tiny
    steps = helpers.trace_mixed(reqs, seed=21)
    places = helpers.wanted_places(steps)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out),
                            "--max-tokens", str(helpers.max_live_tokens(steps))],
                           input="".join(json.dumps(st) + "\n" for st in steps), text=True, capture_output=True, timeout=300)
        assert r.returncode == 0, r.stderr
        assert [w for w in r.stdout.split() if w != "done"] == [str(st["step"]) for st in steps]
        got = {}
        for st in steps:
            if st["step"] in places:
                rows = np.fromfile(out / f"{st['step']}.f32", dtype="<f4").reshape(len(places[st["step"]]), -1)
                got.update(zip(places[st["step"]], rows))
        assert len(got) == sum(len(t) for t in reqs.values())
        if dtype == "float32":
            helpers.compare(got, want, TOL[dtype], "trace_run " + dtype)
        else:
            far = sum(float(np.max(np.abs(row - want[r][pos]))) > TOL[dtype] * float(np.max(np.abs(want[r]))) for (r, pos), row in got.items())
            assert far <= len(got) // 10, f"{far} of {len(got)} rows are far from the plain logits"


def test_greedy_generation_through_the_session(gpu, tiny):
    """Greedy continuation of three prompts through Session.generate (the scheduler, the sampler, graphs): every token
    is the plain implementation's best, or within rounding of it."""
    import hf_cpu_amd.session as S
    name, cfg, d, reqs, _ = tiny
    prompts = [reqs["r1"], reqs["r2"], reqs["r4"]]
    pcfg, w = pg.read_model(d)
    s = S.Session(d, dtype="float32", ctx_max=256, batch=16, page_size=gh.PAGE[name], max_seqs=4)
    gens = s.generate(prompts, temp=0.0, max_tokens=20)
    for g, p in zip(gens, prompts):
        assert len(g.tokens) == 20
        toks = list(p)
        rows = None
        for i, t in enumerate(g.tokens):
            row = pg.forward(pcfg, w, toks)[-1]
            assert row[int(np.argmax(row))] - row[t] <= 1e-4, f"token {i} = {t}, plain picks {int(np.argmax(row))}"
            toks.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_chunks_decoded_token_by_token(gpu, tmp_path, dtype):
    """Chunks of several hundred positions: a decoded token's keys are cut over many waves, counted from its chunk's
    start, in the kernel that also rotates and stores (the layer with keys of its own) and in the one that only attends
    (its reader, with a shorter chunk); two requests decoded together across the border of both chunks."""
    import hf_cpu_amd
    cfg = dict(architecture="Goridra", vocab=300, width=128, logit_softcap=20.0, norm=dict(eps=1e-6), layers=[
        gh.layer(gh.attention(4, 1, 64, 64, 64, 20000.0, 600), gh.dense(128)),
        gh.layer(gh.attention(4, 1, 64, 64, 64, 20000.0, 350, kv_from=0), None)])
    d = gh.make_model_dir(str(tmp_path / "m"), cfg, seed=4, stored="BF16")
    reqs = gh.random_requests(cfg, [733, 1222], seed=2)
    want = gh.plain_logits(d, reqs)
    steps = []
    heads = {r: len(t) - 45 for r, t in reqs.items()}
    for r, t in reqs.items():
        steps.append(helpers._step(len(steps), [(r, t[:heads[r]], [heads[r] - 1])]))
    for i in range(45):
        steps.append(helpers._step(len(steps), [(r, t[heads[r] + i:heads[r] + i + 1], [0]) for r, t in reqs.items()],
                                   list(reqs) if i == 44 else []))
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=helpers.max_live_tokens(steps), max_seqs=2)
    got = helpers.run_trace_in_engine(engine, steps)
    assert len(got) == 2 * 46
    helpers.compare(got, want, TOL[dtype], f"long chunks {dtype}")
    engine.manager.check()


def test_random_weights_and_a_second_configuration_of_the_same_files(gpu, tmp_path):
    """``write_random_model`` makes a folder for this design too, and the engine reads it back; a model whose layers
    all read one layer's keys and values, with one expert and one group, runs as well."""
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    cfg = dict(architecture="Goridra", vocab=90, width=64, logit_softcap=5.0, norm=dict(eps=1e-6), layers=[
        gh.layer(gh.attention(2, 1, 32, 32, 32, 1000.0, 10), gh.moe(1, 1, 1, 1, 16)),
        gh.layer(gh.attention(2, 1, 32, 32, 32, 1000.0, 1000, kv_from=0), None),
        gh.layer(gh.attention(2, 1, 32, 32, 32, 1000.0, 1, kv_from=0), gh.dense(8))])
    # widths that are no multiple of 8 (bf16 matrices that the matrix cores do not take), heads of 20 and 28
    odd = dict(architecture="Goridra", vocab=77, width=100, logit_softcap=50.0, norm=dict(eps=1e-3), layers=[
        gh.layer(gh.attention(3, 1, 20, 28, 10, 300.0, 13), gh.dense(36)),
        gh.layer(gh.attention(3, 1, 20, 28, 10, 300.0, 9, kv_from=0), gh.moe(2, 2, 2, 2, 12))])
    for k, c in enumerate((cfg, odd)):
        d = str(tmp_path / f"m{k}")
        hf_cpu_amd.write_random_model(d, config_from_dict(c), seed=3, dtype="bfloat16")
        pcfg, w = pg.read_model(d)
        toks = [int(t) for t in np.random.default_rng(0).integers(0, c["vocab"], 45)]
        want = pg.forward(pcfg, w, toks)
        for dtype in ("float32", "bfloat16"):
            engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=4, max_tokens=64, max_seqs=1)
            got = engine.step([("a", toks[:31], list(range(31)))]).cpu().numpy()
            assert np.max(np.abs(got - want[:31])) <= TOL[dtype] * np.max(np.abs(want))
            for i in range(31, 45):
                got = engine.step([("a", toks[i:i + 1], [0])]).cpu().numpy()
                assert np.max(np.abs(got[0] - want[i])) <= TOL[dtype] * np.max(np.abs(want))
