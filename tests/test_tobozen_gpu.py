"""Tobozen in the engine against its plain implementation (tests/plain_tobozen.py): each mechanism alone at the
kernels, then whole models in every way of cutting the work.

In bf16 a router's near tie may fall the other way than in float64, which changes a token's output by far more than
rounding. The model tests in bf16 therefore hand the plain implementation the experts that the engine chose, and
check separately that the engine's choice is the plain one wherever the scores are not close.
"""
import math
import types

import numpy as np
import pytest
import torch

import helpers
import plain_tobozen as pt
import tobozen_helpers as th
from test_kernels_gpu import FakeCache, FakeStep, dev, from_value_layout, ints, paged_setup, rounded, to_value_layout

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
# Largest |logit difference| from the float64 plain implementation, as a fraction of the request's largest |logit|.
# fp32: the rounding of the fused multiply-adds and exponentials along a few hundred steps of a recurrence; a lost
# state, a tap too many, a missing term in a softmax or a wrong expert shows as 1e-2 and more.
# bf16: activations and cache rounded to 8 bits of mantissa at every part; in the model of width 40 a value is the sum
# of few products and single roundings show (measured: up to 3.9e-2 at one position, 1.5e-2 at most others).
TOL = {"float32": 3e-5, "bfloat16": 3e-2}
TOL_OF = {("small", "bfloat16"): 6e-2}


def ops_for(ops32, ops16, dtype):
    return ops32 if dtype == torch.float32 else ops16


def state_step(q_lens, slots):
    """What the kernels with per-request state read of a step: request ranges and state rows."""
    starts = np.concatenate([[0], np.cumsum(q_lens)])
    return types.SimpleNamespace(q_start=ints(starts), seq_slot=ints(slots), n_seqs=len(q_lens), max_q_len=int(max(q_lens)),
                                 n_tokens=int(starts[-1]))


# ---- mechanisms alone ----------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,groups", [(40, 4), (5, 1), (5, 5), (256, 4), (320, 2), (1000, 8), (4096, 1), (12288, 3)])
def test_norm_in_groups(ops32, dtype, width, groups):
    rng = np.random.default_rng(width + groups)
    x = (rng.standard_normal((7, width)) * rng.uniform(0.1, 30.0, (7, 1))).astype(np.float32)
    x[:, :width // groups] *= 50.0                       # a run's scale is its own
    w = (1.0 + 0.2 * rng.standard_normal(width)).astype(np.float32)
    out = torch.empty((7, width), dtype=dtype, device="cuda")
    ops32.group_rmsnorm(dev(x), dev(w), 1e-5, groups, out)
    want = pt.group_rms_norm(x.astype(np.float64), w, 1e-5, groups)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert np.max(np.abs(out.float().cpu().numpy() - want) / (np.abs(want) + 1.0)) <= tol
    rows = [6, 0, 3, 3]
    out = torch.empty((4, width), dtype=dtype, device="cuda")
    ops32.group_rmsnorm(dev(x), dev(w), 1e-5, groups, out, rows=ints(rows))
    assert np.max(np.abs(out.float().cpu().numpy() - want[rows]) / (np.abs(want[rows]) + 1.0)) <= tol
    # the gate before the norm (times silu) and after it (times the logistic function), the gate inside wider rows
    for gdt in DTYPES:
        wide = rounded(rng.standard_normal((7, width + 9)), gdt)
        gate = dev(wide, gdt)[:, 4:4 + width]
        for kind, fn in (("silu_before", lambda: pt.group_rms_norm(x * pt.silu(wide[:, 4:4 + width]), w, 1e-5, groups)),
                         ("sigmoid_after", lambda: pt.group_rms_norm(x.astype(np.float64), w, 1e-5, groups) * pt.sigmoid(wide[:, 4:4 + width]))):
            out = torch.empty((7, width), dtype=dtype, device="cuda")
            ops32.group_rmsnorm(dev(x), dev(w), 1e-5, groups, out, gate=gate, gate_kind=kind)
            assert np.max(np.abs(out.float().cpu().numpy() - fn()) / (np.abs(fn()) + 1.0)) <= tol, kind


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,K", [(5, 2), (400, 3), (33, 4), (1300, 4), (7, 1), (64, 8)])
def test_short_convolution_carries_its_last_inputs(ops32, dtype, C, K):
    """Three requests whose tokens come in portions of every size, also shorter than the taps reach back, against the
    convolution of the whole sequences; then a request in a state row that another has used (cleared, as at admission)."""
    rng = np.random.default_rng(C * K)
    lengths = [150, 9, 70]
    seqs = [rounded(rng.standard_normal((n, C)), dtype) for n in lengths]
    taps, bias = rng.standard_normal((C, K)).astype(np.float32), rng.standard_normal(C).astype(np.float32)
    want = [pt.silu(pt.causal_conv(u, taps.astype(np.float64), bias.astype(np.float64))) for u in seqs]
    state = torch.zeros((4, (K - 1) * C + 5), dtype=torch.float32, device="cuda")[:, 5:]
    cuts = [[1, 1, 2, 1, 70, 3, 64, 2, 1, 5], [2, 1, 1, 1, 2, 2], [65, 1, 1, 3]]
    at = [0, 0, 0]
    slots = [2, 0, 3]
    got = [np.zeros_like(u) for u in want]
    for turn in range(max(len(c) for c in cuts)):
        live = [s for s in range(3) if turn < len(cuts[s])]
        rows = np.concatenate([seqs[s][at[s]:at[s] + cuts[s][turn]] for s in live])
        x = torch.zeros((rows.shape[0], C + 3), dtype=dtype, device="cuda")
        x[:, 3:] = dev(rows, dtype)
        out = torch.empty((rows.shape[0], C), dtype=torch.float32, device="cuda")
        step = state_step([cuts[s][turn] for s in live], [slots[s] for s in live])
        ops32.causal_conv(x[:, 3:], dev(taps), dev(bias), state, step, out, activation="silu")
        o, r0 = out.cpu().numpy(), 0
        for s in live:
            n = cuts[s][turn]
            got[s][at[s]:at[s] + n] = o[r0:r0 + n]
            at[s], r0 = at[s] + n, r0 + n
    for s in range(3):
        assert at[s] == lengths[s]
        assert np.max(np.abs(got[s] - want[s])) <= 2e-5, f"request {s}"
    state[0].zero_()
    out = torch.empty((lengths[2], C), dtype=torch.float32, device="cuda")
    ops32.causal_conv(dev(seqs[2], dtype), dev(taps), dev(bias), state, state_step([lengths[2]], [0]), out, activation="silu")
    assert np.max(np.abs(out.cpu().numpy() - want[2])) <= 2e-5


def scan_in_portions(ops, q, k, v, cuts, slots, n_state, call):
    """Runs ``call(step, rows of each request's q, k, v, state, out)`` portion by portion; returns each request's rows."""
    T = [len(x) for x in q]
    state = torch.zeros((max(slots) + 2, n_state), dtype=torch.float32, device="cuda")
    at = [0] * len(q)
    got = [None] * len(q)
    for turn in range(max(len(c) for c in cuts)):
        live = [s for s in range(len(q)) if turn < len(cuts[s])]
        take = {s: slice(at[s], at[s] + cuts[s][turn]) for s in live}
        step = state_step([cuts[s][turn] for s in live], [slots[s] for s in live])
        out = call(step, live, take, state)
        r0 = 0
        for s in live:
            n = cuts[s][turn]
            got[s] = out[r0:r0 + n] if got[s] is None else np.concatenate([got[s], out[r0:r0 + n]])
            at[s], r0 = at[s] + n, r0 + n
    assert at == T
    return got


@pytest.mark.parametrize("H,G,N,P", [(3, 3, 7, 5), (6, 3, 32, 24), (4, 1, 64, 64), (8, 4, 16, 32), (2, 1, 128, 64), (2, 2, 200, 8), (1, 1, 4, 256)])
def test_state_space_recurrence_in_portions(ops32, H, G, N, P):
    """Step sizes through softplus, decays through two exponentials, groups of heads that share B and C, the skip
    term: three requests in portions down to one token against the recurrence over the whole sequences."""
    rng = np.random.default_rng(H * N + P)
    lengths, cuts, slots = [90, 5, 33], [[1, 2, 17, 1, 69], [2, 3], [16, 1, 16]], [1, 3, 0]
    x = [rng.standard_normal((n, H, P)) for n in lengths]
    B = [rng.standard_normal((n, G, N)) * 0.5 for n in lengths]
    C = [rng.standard_normal((n, G, N)) * 0.5 for n in lengths]
    raw = [rounded(rng.standard_normal((n, H)) * 2.0, torch.bfloat16) for n in lengths]
    raw[0][3, 0], raw[0][4, 0] = 60.0, -60.0                      # softplus far from zero on both sides
    dt_bias, A_log, D = rng.standard_normal(H) * 0.5, rng.standard_normal(H) * 0.7 - 1.0, rng.standard_normal(H)
    f32 = lambda a: np.asarray(a, np.float32).astype(np.float64)
    want = [pt.ssm_scan(f32(x[s]), f32(B[s]), f32(C[s]), pt.softplus(raw[s] + f32(dt_bias)), f32(A_log), f32(D)).reshape(lengths[s], -1)
            for s in range(3)]

    def call(step, live, take, state):
        cat = lambda parts, width: dev(np.concatenate([p[take[s]].reshape(-1, width) for s, p in zip(live, [parts[s] for s in live])]))
        T = step.n_tokens
        y = torch.empty((T, H * P), dtype=torch.float32, device="cuda")
        step_size = dev(np.concatenate([raw[s][take[s]] for s in live]), torch.bfloat16)
        ops32.linear_scan(cat(C, G * N), cat(B, G * N), cat(x, H * P), G, N, H, P, state, step, y, step_size=step_size,
                          step_bias=dev(dt_bias), a_log=dev(A_log), skip=dev(D))
        return y.cpu().numpy()
    assert ops32.scan_state_floats(H, N, P) == ops32.lib.hfa_linear_scan_state_floats(H, N, P) >= H * N * P
    got = scan_in_portions(ops32, x, B, C, cuts, slots, ops32.scan_state_floats(H, N, P) + 3, call)
    for s in range(3):
        scale = np.max(np.abs(want[s]))
        assert np.max(np.abs(got[s] - want[s])) <= 2e-5 * scale, f"request {s}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(3, 6, 10), (4, 64, 32), (2, 128, 64), (4, 32, 96), (1, 16, 200)])
def test_linear_attention_recurrence_in_portions(ops32, dtype, H, D, Dv):
    """A fixed decay per head (1, 1/2 and values between), no other scale: portions against the whole."""
    rng = np.random.default_rng(H + D + Dv)
    lengths, cuts, slots = [120, 40], [[2, 1, 50, 3, 64], [40]], [0, 2]
    decay = np.array(([1.0, 0.5, 0.96875, 0.875] * H)[:H])
    q = [rounded(np.abs(rng.standard_normal((n, H, D))) * 0.3, dtype) for n in lengths]
    k = [rounded(np.abs(rng.standard_normal((n, H, D))) * 0.3, dtype) for n in lengths]
    v = [rounded(rng.standard_normal((n, H, Dv)), dtype) for n in lengths]
    want = []
    for s, n in enumerate(lengths):
        o = np.zeros((n, H, Dv))
        for h in range(H):
            S = np.zeros((D, Dv))
            for t in range(n):
                S = decay[h] * S + np.outer(k[s][t, h], v[s][t, h])
                o[t, h] = S.T @ q[s][t, h]
        want.append(o.reshape(n, -1))

    def call(step, live, take, state):
        rows = lambda parts, width: np.concatenate([parts[s][take[s]].reshape(-1, width) for s in live])
        qkv = dev(np.concatenate([rows(q, H * D), rows(k, H * D), rows(v, H * Dv)], axis=1), dtype)      # one matrix, as the mixer holds them
        y = torch.empty((step.n_tokens, H * Dv), dtype=torch.float32, device="cuda")
        ops32.linear_scan(qkv[:, :H * D], qkv[:, H * D:2 * H * D], qkv[:, 2 * H * D:], H, D, H, Dv, state, step, y, decay=dev(decay))
        return y.cpu().numpy()
    assert ops32.scan_state_floats(H, D, Dv) == ops32.lib.hfa_linear_scan_state_floats(H, D, Dv) >= H * D * Dv
    got = scan_in_portions(ops32, q, k, v, cuts, slots, ops32.scan_state_floats(H, D, Dv), call)
    for s in range(2):
        assert np.max(np.abs(got[s] - want[s])) <= 2e-5 * np.max(np.abs(want[s])), f"request {s}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,rot,page,blend", [(3, 3, 10, 6, 4, 8, False), (4, 1, 8, 12, 8, 4, True), (8, 2, 64, 48, 64, 16, True),
                                                    (4, 4, 32, 32, 16, 16, False), (2, 2, 128, 128, 2, 32, True)])
def test_queries_and_keys_normed_whole_rotated_in_pairs_values_blended(ops32, ops16, dtype, H, G, D, Dv, rot, page, blend):
    ops = ops_for(ops32, ops16, dtype)
    rng = np.random.default_rng(H * D + rot)
    T, base, eps = 37, 777.0, 1e-5
    positions = rng.permutation(200)[:T]
    QD, KD, VD = H * D, G * D, G * Dv
    rows = rounded(rng.standard_normal((T, QD + KD + VD)) * 3.0, dtype)
    qw, kw = (1.0 + 0.2 * rng.standard_normal(QD)).astype(np.float32), (1.0 + 0.2 * rng.standard_normal(KD)).astype(np.float32)
    other, lam = rounded(rng.standard_normal((T, VD)), dtype), np.float32(0.3125)
    slot_map = rng.permutation(12 * page)[:T]
    cache = FakeCache(group=0, k=torch.zeros((12 * page, KD), dtype=dtype, device="cuda"),
                      v=torch.zeros((12 * page, VD), dtype=dtype, device="cuda"), page_tokens=page, window=0)
    inv_freq = dev(np.float64(base) ** (-2.0 * np.arange(rot // 2) / rot))
    qkv = dev(rows, dtype)
    keep = torch.zeros((T, VD), dtype=dtype, device="cuda")
    extra = dict(v_blend=dev(np.array([lam])), v_other=dev(other, dtype)) if blend else dict(v_keep=keep)
    ops.qkv_prepare(qkv, ints(positions), inv_freq, rot, "interleaved", H, G, D, Dv, cache, ints(slot_map), q_norm=dev(qw),
                    k_norm=dev(kw), eps=eps, **extra)
    q = pt.rotate_pairs(pt.group_rms_norm(rows[:, :QD], qw, eps, 1).reshape(T, H, D), positions, rot, base).reshape(T, QD)
    k = pt.rotate_pairs(pt.group_rms_norm(rows[:, QD:QD + KD], kw, eps, 1).reshape(T, G, D), positions, rot, base).reshape(T, KD)
    v = rows[:, QD + KD:]
    if blend:
        v = (1.0 - float(lam)) * v + float(lam) * other
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert np.max(np.abs(qkv[:, :QD].float().cpu().numpy() - q)) <= tol * np.max(np.abs(q))
    assert np.max(np.abs(cache.k.float().cpu().numpy()[slot_map] - k)) <= tol * np.max(np.abs(k))
    assert np.max(np.abs(from_value_layout(cache.v.float().cpu().numpy(), page)[slot_map] - v)) <= tol * np.max(np.abs(v))
    if not blend:
        assert np.array_equal(keep.float().cpu().numpy(), rows[:, QD + KD:].astype(np.float32))
    untouched = np.setdiff1d(np.arange(12 * page), slot_map)
    assert not cache.k.float().cpu().numpy()[untouched].any()


def sink_attention(q, k, v, scale):
    """Queries at the last len(q) positions of a sequence of len(k) keys (float64)."""
    n, ql = k.shape[0], q.shape[0]
    full = np.zeros((n,) + q.shape[1:])
    full[n - ql:] = q
    return pt.attend(full, k.astype(np.float64), v.astype(np.float64), scale).reshape(n, q.shape[1], -1)[n - ql:]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,page,lengths,q_lens", [
    (4, 2, 16, 8, [1, 5, 24, 25, 130, 203], [1, 3, 24, 2, 1, 60]),           # plain kernels: a head of 16
    (8, 2, 64, 16, [700, 96, 97, 333, 64], [100, 96, 1, 17, 1]),             # matrix cores: portions beside decoded tokens
    (8, 4, 32, 16, [2100, 1500, 64, 65, 1], [1, 1, 1, 1, 1]),                # decoded tokens far into long sequences: keys cut into chunks
    (28, 4, 128, 16, [2100, 1025], [1, 1]),
    (4, 1, 64, 64, [600], [600]),                                            # one prompt, whole
    (8, 2, 128, 16, [1500], [1500]),                                         # few blocks: a tile's keys cut over blocks
    (8, 2, 64, 16, [2000, 90], [400, 90]),                                   # a portion late in a prompt
])
def test_attention_with_one_more_term_in_the_softmax(ops32, ops16, dtype, H, G, D, page, lengths, q_lens):
    ops = ops_for(ops32, ops16, dtype)
    rng = np.random.default_rng(H + D + len(lengths))
    ks, vs, cache, table = paged_setup(rng, lengths, G, D, page, dtype)
    qs, positions, slots, wants = [], [], [], []
    scale = 0.6 / math.sqrt(D)                 # scores near zero: the added term is a large share of the denominator
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q = rng.standard_normal((ql, H, D)).astype(np.float32)
        wants.append(sink_attention(rounded(q, dtype), rounded(ks[s], dtype), rounded(vs[s], dtype), scale))
        qs.append(q)
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * D)
    out = torch.empty((q.shape[0], H * D), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops.paged_attention(dev(q, dtype), H, G, D, cache, step, 0, scale, out, sink=True)
    err = np.max(np.abs(out.float().cpu().numpy() - want))
    assert err <= (2e-5 if dtype == torch.float32 else 0.02), f"max |diff| {err:.3e}"
    if min(lengths) <= 100:                    # (among thousands of keys one more term is a small share)
        plain_softmax = torch.empty_like(out)
        ops.paged_attention(dev(q, dtype), H, G, D, cache, step, 0, scale, plain_softmax)
        assert np.max(np.abs(plain_softmax.float().cpu().numpy() - want)) > 0.05, "without the term the result must differ"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,page,n,ql", [(4, 2, 16, 16, 8, 300, 1), (4, 2, 16, 16, 8, 300, 40), (8, 2, 64, 64, 16, 1500, 1), (8, 2, 64, 64, 16, 1500, 200),
                                               (8, 2, 64, 48, 16, 900, 1), (8, 2, 64, 48, 16, 900, 64), (4, 4, 32, 32, 16, 2500, 1)])
def test_a_key_far_away_among_hundreds_and_scores_far_below_zero(ops32, ops16, dtype, H, G, D, Dv, page, n, ql):
    """One key near the start matches every query far better than all others and carries a value of its own: it takes
    the whole output, in a decoded token and in a prompt portion. With every score far below zero the added term takes
    the whole weight and the output is zero (a softmax without it would return an average of the values)."""
    ops = ops_for(ops32, ops16, dtype)
    scale = 1.0 / math.sqrt(D)
    direction = np.ones(D, np.float32) / math.sqrt(D)
    for case in ("far key", "all below zero"):
        rng = np.random.default_rng(n + ql)
        k = (0.1 * rng.standard_normal((n, G, D))).astype(np.float32)
        v = rng.standard_normal((n, G, Dv)).astype(np.float32)
        q = (0.1 * rng.standard_normal((ql, H, D)) + 4.0 * direction).astype(np.float32)
        if case == "far key":
            k[3] = 60.0 * direction
            v[3] = 7.0
        else:
            k -= 160.0 * direction                       # every score about -640 / sqrt(D): -80 and below
        blocks = -(-n // page)
        perm = rng.permutation(blocks + 2)
        table = np.zeros((1, blocks + 1), np.int32)
        table[0, :blocks] = perm[:blocks]
        kc = np.zeros(((blocks + 2) * page, G * D), np.float32)
        vc = np.zeros(((blocks + 2) * page, G * Dv), np.float32)
        for j in range(n):
            row = table[0, j // page] * page + j % page
            kc[row], vc[row] = k[j].reshape(-1), v[j].reshape(-1)
        cache = FakeCache(group=0, k=dev(kc, dtype), v=dev(to_value_layout(vc, page), dtype), page_tokens=page, window=0)
        out = torch.empty((ql, H * Dv), dtype=dtype, device="cuda")
        step = FakeStep(ints(list(range(n - ql, n))), ints([0] * ql), ints(table), None)
        ops.paged_attention(dev(q.reshape(ql, -1), dtype), H, G, D, cache, step, 0, scale, out, v_head_dim=Dv, sink=True)
        got = out.float().cpu().numpy().reshape(ql, H, Dv)
        want = sink_attention(rounded(q, dtype), rounded(k, dtype), rounded(v, dtype), scale)
        assert np.max(np.abs(got - want)) <= (2e-5 if dtype == torch.float32 else 0.03), case
        if case == "far key":
            assert np.all(np.abs(got - 7.0) < 0.1), "the key at position 3 should take the output"
        else:
            assert np.all(np.abs(got) < 1e-6), "the term of score 0 should take the whole weight"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,F,E,top,limit", [(1, 40, 12, 5, 2, 0.5), (7, 256, 80, 10, 1, 1.25), (300, 256, 64, 4, 4, 2.0), (33, 128, 32, 16, 3, 7.0),
                                               (2100, 256, 32, 8, 2, 1.0), (64, 64, 16, 1, 1, 0.25), (5, 256, 96, 6, 2, 1.0),
                                               (9, 72, 64, 3, 1, 0.5), (1200, 512, 192, 4, 2, 1.5), (40, 80, 64, 4, 2, 1.0), (700, 144, 96, 3, 1, 2.0)])
def test_router_and_gated_experts_weighted_on_their_input(ops32, ops16, dtype, T, W, F, E, top, limit):
    """Sigmoid scores, the best experts, the scores themselves as weights, and the weight inside the expert: the
    bounds at ``limit`` cut differently for ``expert(w h)`` than for ``w expert(h)``."""
    ops = ops_for(ops32, ops16, dtype)
    rng = np.random.default_rng(T + W + E)
    h = rounded(rng.standard_normal((T, W)), dtype)
    router = rounded(rng.standard_normal((E, W)) * 1.5 / math.sqrt(W), dtype)
    w = {"router": router}
    for e in range(E):
        w[f"e{e}.gate"] = rounded(rng.standard_normal((F, W)) * 2.0 / math.sqrt(W), dtype)
        w[f"e{e}.up"] = rounded(rng.standard_normal((F, W)) * 2.0 / math.sqrt(W), dtype)
        w[f"e{e}.down"] = rounded(rng.standard_normal((W, F)) / math.sqrt(F), dtype)
    z = h @ router.T
    logits = dev(z)
    ids, wts = ops.moe_route(logits, top, 1, 1, "sigmoid", False, 1.0)
    ids_h, wts_h = ids.cpu().numpy(), wts.cpu().numpy()
    want_ids, want_w = pt.route(z.astype(np.float32).astype(np.float64), top)
    assert np.array_equal(np.sort(ids_h, axis=1), np.sort(want_ids, axis=1)) or dtype == torch.bfloat16
    assert np.max(np.abs(wts_h - np.take_along_axis(pt.sigmoid(z), ids_h.astype(np.int64), axis=1))) <= 1e-6
    f = dict(expert=dict(ff=F, limit=limit), router=dict(experts=E, top=top))
    want, _ = pt.moe_ff(h, w, "", f, choices=ids_h)
    x = torch.zeros((T, W), dtype=torch.float32, device="cuda")
    gates = dev(np.stack([w[f"e{e}.gate"] for e in range(E)]), dtype)
    ups = dev(np.stack([w[f"e{e}.up"] for e in range(E)]), dtype)
    w_down = dev(np.stack([w[f"e{e}.down"] for e in range(E)]), dtype)
    # gate rows before up rows (the activation is a kernel of its own), and, where the size allows, in blocks of 32 and 32
    # (the activation in the up product's last lines); the matrix-core kernels and the plain one
    layouts = [(torch.cat([gates, ups], 1), False)] + ([(ops.interleave_experts(gates, ups), True)] if F % 32 == 0 else [])
    for w_up, interleaved in layouts:
        for plain_kernels in (False, True):
            x.zero_()
            ops.force_plain_gemm = plain_kernels
            try:
                ops.moe_experts(dev(h, dtype), ids, wts, w_up, w_down, None, x, gated=(1.702, limit, 1.0, interleaved))
            finally:
                ops.force_plain_gemm = False
            err = np.max(np.abs(x.cpu().numpy() - want)) / np.max(np.abs(want))
            assert err <= (1e-5 if dtype == torch.float32 else 1e-2), f"interleaved={interleaved} plain={plain_kernels}: {err:.3e}"


# ---- whole models ---------------------------------------------------------------------------------------------------

LENGTHS = {"small": [1, 2, 3, 23, 24, 57, 130], "cores": [3, 48, 49, 97, 161, 230]}


@pytest.fixture(scope="module", params=["small", "cores"])
def tiny(request, tmp_path_factory):
    name = request.param
    cfg = th.CONFIGS[name]
    d = th.make_model_dir(str(tmp_path_factory.mktemp("tobozen_" + name)), cfg, seed=len(name), stored=th.STORED[name])
    reqs = th.random_requests(cfg, LENGTHS[name], seed=7)
    return name, cfg, d, reqs, th.plain_logits(d, reqs)


def engine_for(model_dir, dtype, name, max_tokens, max_seqs=4, graphs=True):
    import hf_cpu_amd
    return hf_cpu_amd.load_engine(model_dir, dtype=dtype, page_tokens=th.PAGE[name], max_tokens=max_tokens,
                                  max_seqs=max_seqs, graphs=graphs)


def run_against_plain(name, d, reqs, want, dtype, steps, what, graphs=True):
    """Runs the trace; in bf16 with the engine's choice of experts handed to the plain implementation, after checking
    that the choice is the plain one wherever the plain scores are 0.02 or more apart."""
    engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps), graphs=graphs and dtype == "float32")
    if dtype == "float32":
        got = helpers.run_trace_in_engine(engine, steps)
    else:
        with th.record_choices(engine) as rec:
            got = helpers.run_trace_in_engine(engine, steps)
        cfg, w = pt.read_model(d)
        want = {}
        for r, toks in reqs.items():
            margins, mine = {}, rec.chosen.get(r, {})
            want[r] = th.forward_with_choices(cfg, w, toks, mine, margins)
            assert set(mine) == set(margins), f"{what}: request {r}: the router did not run once for every token and layer"
            clear = [key for key, (gap, _) in margins.items() if gap >= 0.02]
            wrong = [key for key in clear if not margins[key][1]]
            assert not wrong, f"{what}: request {r}: at (layer, position) {wrong[:5]} the engine chose other experts than the " \
                              "plain router although the scores are apart"
    worst = helpers.compare(got, want, TOL_OF.get((name, dtype), TOL[dtype]), what)
    engine.manager.check()
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)
    return engine, got, worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cutting", ["whole", "tail", "portions", "mixed"])
def test_cuttings(gpu, tiny, dtype, cutting):
    """Whole prompts; most of a prompt and then token by token; portions of changing size down to two tokens; up to
    four requests live, portions beside single tokens, pages and state rows used again."""
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
            assert err <= 3e-5 * max(1.0, float(np.max(np.abs(row)))), f"{name}: {key}: cuttings differ by {err:.3e}"


def test_a_batch_of_unequal_requests_against_each_alone(gpu, tiny):
    name, cfg, d, reqs, want = tiny
    engine = engine_for(d, "float32", name, 64 * len(reqs) + sum(len(t) for t in reqs.values()), max_seqs=len(reqs))
    together = engine.step([(r, toks, list(range(len(toks)))) for r, toks in reqs.items()]).cpu().numpy()
    at = 0
    for r, toks in reqs.items():
        engine.release(r)
        alone = engine.step([(r + "'", toks, list(range(len(toks))))]).cpu().numpy()
        engine.release(r + "'")
        assert np.max(np.abs(alone - together[at:at + len(toks)])) <= 3e-5 * np.max(np.abs(want[r]))
        assert np.max(np.abs(alone - want[r])) <= TOL["float32"] * np.max(np.abs(want[r]))
        at += len(toks)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_small_pool(gpu, tiny, dtype):
    """Three requests decoded token by token together from their second token on, in a pool that holds them and no
    more, then three more in the pages and state rows that they gave back: what the first left there must be gone."""
    name, cfg, d, reqs, want = tiny
    long = {r: t for r, t in reqs.items() if len(t) >= 57}
    names = list(long)[:3]
    order = [names, names[::-1]]                    # the second turn's requests land in other state rows than the first's
    steps = []
    for turn in range(2):
        ids = {r: f"{r}/{turn}" for r in names}
        steps.append(helpers._step(len(steps), [(ids[r], long[r][:2], [0, 1]) for r in order[turn]]))
        for i in range(2, max(len(long[r]) for r in names)):
            live = [r for r in order[turn] if i < len(long[r])]
            steps.append(helpers._step(len(steps), [(ids[r], long[r][i:i + 1], [0]) for r in live],
                                       [ids[r] for r in live if i == len(long[r]) - 1]))
    reqs2 = {f"{r}/{turn}": long[r] for r in names for turn in range(2)}
    want2 = {f"{r}/{turn}": want[r] for r in names for turn in range(2)}
    engine = None
    engine, got, _ = run_against_plain(name, d, reqs2, want2, dtype, steps, f"{name} {dtype} long decoding")
    assert all(p.reused > 0 for p in engine.manager.pools)
    if dtype == "float32":
        assert engine.graph_replays > 0, "decode steps were meant to replay captured graphs"


def test_trace_replay_program(gpu, tiny, tmp_path):
    """bin/trace_run as a user calls it (pages of 16, four state rows, a pool for the live requests only): a mixed
    trace in fp32 against the plain implementation; in bf16 against the engine in this process on the same trace (which
    ``test_cuttings`` holds against the plain implementation with the engine's choice of experts: a near tie that falls
    the other way changes the states, and with them every later token of the request)."""
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
            engine = engine_for(d, dtype, "cores", helpers.max_live_tokens(steps))      # pages of 16, as the program's
            same = helpers.run_trace_in_engine(engine, steps)
            for key, row in got.items():
                assert np.max(np.abs(row - same[key])) <= 1e-5 * np.max(np.abs(same[key])), f"{key}: the program and the engine differ"


def test_greedy_generation_through_the_session(gpu, tiny):
    """Greedy continuation of three prompts through Session.generate (the scheduler, the sampler, graphs): every token
    is the plain implementation's best, or within rounding of it."""
    import hf_cpu_amd.session as S
    name, cfg, d, reqs, _ = tiny
    prompts = [reqs["r3"], reqs["r4"], reqs["r5"]]
    pcfg, w = pt.read_model(d)
    s = S.Session(d, dtype="float32", ctx_max=256, batch=16, page_size=th.PAGE[name], max_seqs=4)
    gens = s.generate(prompts, temp=0.0, max_tokens=20)
    for g, p in zip(gens, prompts):
        assert len(g.tokens) == 20
        toks = list(p)
        for i, t in enumerate(g.tokens):
            row = pt.forward(pcfg, w, toks)[-1]
            assert row[int(np.argmax(row))] - row[t] <= 1e-4 * max(1.0, float(np.max(np.abs(row)))), \
                f"token {i} = {t}, plain picks {int(np.argmax(row))}"
            toks.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_decoded_token_by_token(gpu, tmp_path, dtype):
    """Two requests of 700 and 1,300 tokens: the prompt in two portions (the second begins in the middle of a page),
    then 45 tokens decoded together; attention cuts the keys of a decoded token over many waves, the states have been
    carried over a thousand steps."""
    import hf_cpu_amd
    cfg = dict(architecture="Tobozen", vocab=300, width=128, norm=dict(eps=1e-6, groups=2), layers=[
        th.layer(th.attention(4, 1, 64, 64, 64, 30000.0, v_mix=True), th.moe(4, 1, 64, 1.0)),
        th.layer(th.mamba2(2, 64, 32, 2, 4, 1), None),
        th.layer(th.lightning(2, 64, 64, [0.99609375, 0.9375]), None),
        th.layer(th.attention(4, 1, 64, 64, 64, 30000.0, v_mix=True), None)])
    d = th.make_model_dir(str(tmp_path / "m"), cfg, seed=4, stored="BF16")
    reqs = th.random_requests(cfg, [700, 1300], seed=2)
    want = th.plain_logits(d, reqs)
    steps = []
    heads = {r: len(t) - 45 for r, t in reqs.items()}
    for r, t in reqs.items():
        steps.append(helpers._step(len(steps), [(r, t[:heads[r] - 201], [heads[r] - 202])]))
        steps.append(helpers._step(len(steps), [(r, t[heads[r] - 201:heads[r]], [0, 200])]))
    for i in range(45):
        steps.append(helpers._step(len(steps), [(r, t[heads[r] + i:heads[r] + i + 1], [0]) for r, t in reqs.items()],
                                   list(reqs) if i == 44 else []))
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=helpers.max_live_tokens(steps), max_seqs=2)
    got = helpers.run_trace_in_engine(engine, steps)
    assert len(got) == 2 * 48
    helpers.compare(got, want, TOL[dtype], f"long prompts {dtype}")
    engine.manager.check()


def test_random_weights_and_other_orders_of_layers(gpu, tmp_path):
    """``write_random_model`` makes a folder for this design too, and the engine reads it back: a model that begins with
    linear attention and ends with a state-space layer, one expert, one head; and one with widths that are no multiple
    of 8."""
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    cfg = dict(architecture="Tobozen", vocab=90, width=64, norm=dict(eps=1e-6, groups=8), layers=[
        th.layer(th.lightning(1, 32, 32, [0.75]), th.moe(1, 1, 16, 1.0)),
        th.layer(th.attention(2, 1, 32, 32, 32, 1000.0), None),
        th.layer(th.mamba2(1, 32, 8, 1, 2, 1), th.moe(2, 2, 8, 1.0))])
    odd = dict(architecture="Tobozen", vocab=77, width=100, norm=dict(eps=1e-3, groups=5), layers=[
        th.layer(th.mamba2(5, 4, 3, 5, 3, 2), th.moe(3, 2, 12, 0.3)),
        th.layer(th.attention(3, 1, 20, 28, 10, 300.0, v_mix=True), None),
        th.layer(th.attention(3, 1, 10, 28, 10, 300.0, v_mix=True), th.moe(2, 1, 20, 2.0))])
    for k, c in enumerate((cfg, odd)):
        d = str(tmp_path / f"m{k}")
        hf_cpu_amd.write_random_model(d, config_from_dict(c), seed=3, dtype="bfloat16")
        pcfg, w = pt.read_model(d)
        toks = [int(t) for t in np.random.default_rng(0).integers(0, c["vocab"], 45)]
        want = pt.forward(pcfg, w, toks)
        for dtype in ("float32", "bfloat16"):
            engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=4, max_tokens=64, max_seqs=1)
            got = engine.step([("a", toks[:31], list(range(31)))]).cpu().numpy()
            far = np.max(np.abs(got - want[:31]), axis=1) > TOL[dtype] * np.max(np.abs(want))
            assert far.sum() <= (0 if dtype == "float32" else 3)             # (bf16: a router's near tie may fall the other way)
            for i in range(31, 45):
                got = engine.step([("a", toks[i:i + 1], [0])]).cpu().numpy()
                assert dtype == "bfloat16" or np.max(np.abs(got[0] - want[i])) <= TOL[dtype] * np.max(np.abs(want))


def test_a_file_may_hold_the_weights_that_are_never_read(gpu, tmp_path):
    """The second norm of a layer without a feed-forward and the first mixing layer's blend are read by nothing: a
    folder that holds them loads and computes what a folder without them does."""
    import hf_cpu_amd
    cfg = th.SMALL
    w = th.make_weights(cfg, seed=9)
    toks = [int(t) for t in np.random.default_rng(3).integers(0, cfg["vocab"], 20)]
    outs = []
    for k, extra in enumerate(({}, {"l1.norm2": np.full(cfg["width"], 3.0, np.float32), "l4.norm2": np.ones(cfg["width"], np.float32)})):
        wk = dict(w, **extra)
        if k == 0:
            del wk["l2.mix.vmix"]
        d = th.make_model_dir(str(tmp_path / f"m{k}"), cfg, seed=0, weights=wk)
        engine = hf_cpu_amd.load_engine(d, dtype="float32", page_tokens=8, max_tokens=64, max_seqs=1)
        outs.append(engine.step([("a", toks, list(range(len(toks))))]).cpu().numpy())
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("seed", range(6))
def test_configurations_drawn_at_random(gpu, tmp_path, seed):
    """Layers of any kind in any order with sizes drawn at random (even seeds: sizes for the matrix cores): a prompt, a portion
    that starts in the middle of a page, then single tokens, in fp32 and in bf16 (with the engine's choice of experts)."""
    import hf_cpu_amd
    rng = np.random.default_rng(100 + seed)
    cfg = th.random_config(rng, big=seed % 2 == 0)
    d = th.make_model_dir(str(tmp_path / "m"), cfg, seed=seed, stored="BF16" if seed % 2 == 0 else "F32")
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 110)]
    pcfg, w = pt.read_model(d)
    steps = [helpers._step(0, [("a", toks[:55], range(55))]), helpers._step(1, [("a", toks[55:88], range(33))])]
    steps += [helpers._step(2 + i, [("a", toks[88 + i:89 + i], [0])], ["a"] if i == 21 else []) for i in range(22)]
    for dtype in ("float32", "bfloat16"):
        engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=128, max_seqs=2, graphs=dtype == "float32")
        if dtype == "float32":
            got, want = helpers.run_trace_in_engine(engine, steps), pt.forward(pcfg, w, toks)
        else:
            with th.record_choices(engine) as rec:
                got = helpers.run_trace_in_engine(engine, steps)
            want = th.forward_with_choices(pcfg, w, toks, rec.chosen.get("a", {}))
        helpers.compare(got, {"a": want}, TOL[dtype] if dtype == "float32" else 6e-2, f"random configuration {seed} {dtype}: {cfg}")
