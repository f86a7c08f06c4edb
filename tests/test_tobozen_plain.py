"""The plain implementation of the Tobozen design (tests/plain_tobozen.py) held against library routines, second
derivations and special cases, and the configuration reader and plan of the package. All on the CPU."""
import copy
import math

import numpy as np
import pytest
import torch

import plain
import plain_tobozen as pt
import tobozen_helpers as th


def test_norm_in_groups():
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal((5, 24)), rng.standard_normal(24)
    assert np.allclose(pt.group_rms_norm(x, w, 1e-6, 1), plain.rmsnorm(x, w, 1e-6), atol=1e-12)
    y = pt.group_rms_norm(x, np.ones(24), 0.0, 4).reshape(5, 4, 6)
    assert np.allclose((y * y).mean(axis=-1), 1.0)
    # a run's scale is its own: making another run large changes nothing in this one
    x2 = x.copy()
    x2[:, 6:12] *= 100.0
    assert np.allclose(pt.group_rms_norm(x2, w, 1e-6, 4)[:, :6], pt.group_rms_norm(x, w, 1e-6, 4)[:, :6])
    # eps is inside the root
    assert np.allclose(pt.group_rms_norm(np.zeros((1, 4)) + 3.0, np.ones(4), 16.0, 1), 3.0 / 5.0)


def test_short_convolution_against_the_library():
    rng = np.random.default_rng(1)
    u, taps, bias = rng.standard_normal((9, 3)), rng.standard_normal((3, 4)), rng.standard_normal(3)
    got = pt.causal_conv(u, taps, bias)
    for c in range(3):
        want = np.convolve(u[:, c], taps[c, ::-1])[:9] + bias[c]          # the last tap is the current token's
        assert np.allclose(got[:, c], want)
    assert np.allclose(got[0], bias + taps[:, -1] * u[0])                   # zeros before the start


def test_state_space_recurrence_against_its_sum_form():
    """y_t = sum over s <= t of (prod of the decays after s up to t) dt_s (B_s . C_t) x_s + D x_t."""
    rng = np.random.default_rng(2)
    T, H, P, G, N = 11, 4, 3, 2, 5
    x, B, C = rng.standard_normal((T, H, P)), rng.standard_normal((T, G, N)), rng.standard_normal((T, G, N))
    dt, A_log, D = rng.random((T, H)) + 0.1, rng.standard_normal(H), rng.standard_normal(H)
    got = pt.ssm_scan(x, B, C, dt, A_log, D)
    for h in range(H):
        g = h // (H // G)
        loga = -np.exp(A_log[h]) * dt[:, h]
        for t in range(T):
            want = D[h] * x[t, h]
            for s in range(t + 1):
                want = want + np.exp(loga[s + 1:t + 1].sum()) * dt[s, h] * (B[s, g] @ C[t, g]) * x[s, h]
            assert np.allclose(got[t, h], want)


def test_softplus_and_silu():
    z = np.array([-800.0, -3.0, 0.0, 2.0, 900.0])
    assert np.allclose(pt.softplus(z), [0.0, math.log1p(math.exp(-3.0)), math.log(2.0), math.log1p(math.exp(2.0)), 900.0])
    assert np.allclose(pt.silu(np.array([0.0, 1.0])), [0.0, 1.0 / (1.0 + math.exp(-1.0))])


def test_rotation_in_neighbouring_pairs():
    rng = np.random.default_rng(3)
    v = rng.standard_normal((6, 2, 10))
    pos = np.array([0, 1, 2, 7, 100, 1000])
    r = pt.rotate_pairs(v, pos, 6, 50.0)
    assert np.allclose(r[0], v[0])                                        # position 0: no rotation
    assert np.allclose(r[..., 6:], v[..., 6:])                            # dimensions beyond rot.dims pass
    assert np.allclose((r ** 2).sum(-1), (v ** 2).sum(-1))
    # dimension 0 pairs with 1, not with 3: a vector along dimension 0 stays in the plane (0, 1), by the angle pos * 1
    e = np.zeros((1, 1, 10))
    e[..., 0] = 1.0
    out = pt.rotate_pairs(e, [2], 6, 50.0)[0, 0]
    assert np.allclose(out[:2], [math.cos(2.0), math.sin(2.0)]) and np.allclose(out[2:], 0.0)
    # pair i turns by pos * base^(-2i/dims)
    e = np.zeros((1, 1, 10))
    e[..., 4] = 1.0
    out = pt.rotate_pairs(e, [3], 6, 50.0)[0, 0]
    a = 3.0 * 50.0 ** (-4.0 / 6.0)
    assert np.allclose(out[4:6], [math.cos(a), math.sin(a)])
    # scores depend on the distance only
    q, k = rng.standard_normal((1, 1, 6)), rng.standard_normal((1, 1, 6))
    d1 = (pt.rotate_pairs(q, [9], 6, 50.0) * pt.rotate_pairs(k, [4], 6, 50.0)).sum()
    d2 = (pt.rotate_pairs(q, [105], 6, 50.0) * pt.rotate_pairs(k, [100], 6, 50.0)).sum()
    assert np.allclose(d1, d2)


def test_attention_with_one_more_term_against_the_library():
    """A key of zeros with a value of zeros that every query sees is the term of score 0 that has no value."""
    rng = np.random.default_rng(4)
    T, H, G, D, Dv = 9, 4, 2, 6, 5
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, G, D)), rng.standard_normal((T, G, Dv))
    got = pt.attend(q, k, v, 0.7).reshape(T, H, Dv)
    tq = torch.from_numpy(q).permute(1, 0, 2)
    tk = torch.from_numpy(np.concatenate([np.zeros((1, G, D)), k])).permute(1, 0, 2).repeat_interleave(H // G, 0)
    tv = torch.from_numpy(np.concatenate([np.zeros((1, G, Dv)), v])).permute(1, 0, 2).repeat_interleave(H // G, 0)
    mask = torch.ones(T, T + 1, dtype=torch.bool).tril(1)
    mask[:, 0] = True
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=0.7).permute(1, 0, 2).numpy()
    assert np.allclose(got, want, atol=1e-12)
    p = pt.sink_softmax(np.array([[-1000.0, -1001.0], [1000.0, 999.0], [0.0, -np.inf]]))
    assert np.allclose(p[0], 0.0) and np.allclose(p[1].sum(), 1.0) and np.allclose(p[2], [0.5, 0.0])


def test_linear_attention_against_its_sum_form():
    rng = np.random.default_rng(5)
    cfg = dict(heads=2, dim=3, vdim=4, decay=[0.5, 1.0])
    E, T = 6, 8
    w = {"q": rng.standard_normal((6, E)), "k": rng.standard_normal((6, E)), "v": rng.standard_normal((8, E)),
         "g": rng.standard_normal((8, E)), "norm": rng.standard_normal(8), "o": rng.standard_normal((E, 8))}
    h = rng.standard_normal((T, E))
    got = pt.lightning(h, w, "", cfg, 1e-6)
    q, k = pt.silu(h @ w["q"].T).reshape(T, 2, 3), pt.silu(h @ w["k"].T).reshape(T, 2, 3)
    v = pt.silu(h @ w["v"].T).reshape(T, 2, 4)
    o = np.zeros((T, 2, 4))
    for hd in range(2):
        for t in range(T):
            for s in range(t + 1):
                o[t, hd] += cfg["decay"][hd] ** (t - s) * (q[t, hd] @ k[s, hd]) * v[s, hd]
    want = (plain.rmsnorm(o.reshape(T, 8), w["norm"], 1e-6) * pt.sigmoid(h @ w["g"].T)) @ w["o"].T
    assert np.allclose(got, want)


def test_router_and_experts():
    z = np.array([[0.1, 2.0, -1.0, 2.0, 0.5], [-3.0, -2.0, -2.5, -9.0, -2.0]])
    ids, wts = pt.route(z, 2)
    assert ids.tolist() == [[1, 3], [1, 4]]                               # the lower index among equals
    assert np.allclose(wts, pt.sigmoid(np.array([[2.0, 2.0], [-2.0, -2.0]])))   # the scores themselves, not renormalised
    rng = np.random.default_rng(6)
    gate, up, down = rng.standard_normal((4, 3)), rng.standard_normal((4, 3)), rng.standard_normal((3, 4))
    h = rng.standard_normal(3)
    g, u = gate @ h, up @ h
    assert np.allclose(pt.expert(h, gate, up, down, 1e9), down @ (g / (1 + np.exp(-1.702 * g)) * (u + 1)))
    # the gate half is bounded above only, the up half on both sides
    big = pt.expert(1e6 * h, gate, up, down, 2.0)
    gl, ul = np.minimum(1e6 * g, 2.0), np.clip(1e6 * u, -2.0, 2.0)
    assert np.allclose(big, down @ (gl / (1 + np.exp(-1.702 * gl)) * (ul + 1)))
    # the weight scales the input: with one expert chosen the layer is expert(w h), which is not w expert(h)
    w = {"router": rng.standard_normal((2, 3)), "e0.gate": gate, "e0.up": up, "e0.down": down,
         "e1.gate": gate, "e1.up": up, "e1.down": down}
    f = dict(expert=dict(ff=4, limit=1e9), router=dict(experts=2, top=1))
    out, zz = pt.moe_ff(h[None], w, "", f)
    s = pt.sigmoid(zz[0]).max()
    assert np.allclose(out[0], pt.expert(s * h, gate, up, down, 1e9)) and not np.allclose(out[0], s * pt.expert(h, gate, up, down, 1e9))


@pytest.fixture(scope="module")
def small():
    cfg = th.SMALL
    return cfg, {k: np.asarray(v, np.float64) for k, v in th.make_weights(cfg, 3).items()}


def test_a_prefix_has_the_logits_of_the_whole(small):
    cfg, w = small
    toks = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 30)]
    whole = pt.forward(cfg, w, toks)
    assert np.allclose(pt.forward(cfg, w, toks[:13]), whole[:13], atol=1e-9)


def test_layers_whose_output_projections_are_zero_leave_the_embedding(small):
    cfg, w = small
    w = dict(w)
    for name in w:
        if name.endswith("mix.o") or name.endswith(".down"):
            w[name] = np.zeros_like(w[name])
    toks = [5, 9, 77]
    want = pt.group_rms_norm(w["embed"][toks], w["final.norm"], cfg["norm"]["eps"], cfg["norm"]["groups"]) @ w["embed"].T
    assert np.allclose(pt.forward(cfg, w, toks), want)


def test_values_are_mixed_with_the_first_mixing_layers(small):
    """With its blend at 1 the later mixing layer attends over the first one's values alone: its own value projection
    no longer matters, while the first mixing layer's blend is never read."""
    cfg, w = small
    toks = [int(t) for t in np.random.default_rng(1).integers(0, cfg["vocab"], 12)]
    base = pt.forward(cfg, w, toks)
    w2 = dict(w)
    w2["l2.mix.vmix"] = np.float64(123.0)                                   # the first mixing layer's: unused
    assert np.allclose(pt.forward(cfg, w2, toks), base)
    w3 = dict(w)
    w3["l4.mix.vmix"] = np.float64(1.0)
    a = pt.forward(cfg, w3, toks)
    w3["l4.mix.v"] = w3["l4.mix.v"] * 3.0
    assert np.allclose(pt.forward(cfg, w3, toks), a) and not np.allclose(a, base)


# ---- the package's configuration reader and plan ----------------------------------------------------------------

def test_configuration_and_plan():
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.kernels.ops import Ops
    from hf_cpu_amd.parts.base import FixedState, PagedKV
    for name, cfg in th.CONFIGS.items():
        c = config_from_dict(cfg)
        assert c.width == cfg["width"] and len(c.layers) == len(cfg["layers"]) and c.to_dict() == cfg
        model = hf_cpu_amd.Model.from_config(c)
        declared = {s.name: tuple(s.shape) for s in model.param_specs() if not s.optional or s.name.endswith("vmix")}
        made = {k: tuple(np.shape(v)) for k, v in th.make_weights(cfg, 0).items()}
        assert declared == made
        needs = model.cache_needs()
        for lc, need in zip(cfg["layers"], needs):
            m = lc["mixer"]
            if lc["type"] == "attention":
                assert need == PagedKV(m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"])
            elif lc["type"] == "lightning":
                assert need == FixedState(Ops.scan_state_floats(m["heads"], m["dim"], m["vdim"]))
                assert need.n_floats >= m["heads"] * m["dim"] * m["vdim"]
            else:
                channels = m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
                assert need == FixedState(Ops.scan_state_floats(m["heads"], m["state"], m["vdim"]) + (m["conv"] - 1) * channels)
        mixes = [lay.mixer.v_mix for lay in model.layers if hasattr(lay.mixer, "v_mix")]
        assert [v for v in mixes if v] == ["first"] + ["blend"] * (len([v for v in mixes if v]) - 1)


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="conv"), "not supported"),
    (lambda c: c["layers"][3]["mixer"].update(groups=2), "multiple"),
    (lambda c: c["layers"][3]["mixer"].update(norm_groups=4), "equal runs"),
    (lambda c: c["layers"][4]["mixer"].update(vdim=8), "mixed"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5, 0.5]), "decay"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=12), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "choices"),
    (lambda c: c["norm"].update(groups=3), "equal runs"),
    (lambda c: c["layers"][5]["mixer"].pop("state"), "state"),
])
def test_configuration_errors_name_what_is_wrong(change, word):
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.status import EngineError
    cfg = copy.deepcopy(th.SMALL)
    change(cfg)
    with pytest.raises(EngineError) as e:
        config_from_dict(cfg)
    assert word in str(e.value.msg)
