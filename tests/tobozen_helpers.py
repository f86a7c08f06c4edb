"""Shared by the Tobozen tests: small configurations that differ in every size and option, weights that give
activations of order one, model folders, and the plain implementation's logits (optionally with the experts that the
engine chose, see ``goridra_helpers.record_choices``, which works for every mixture-of-experts part)."""
import json
import math
import os

import numpy as np

import helpers
import plain_tobozen as pt
from goridra_helpers import record_choices          # noqa: F401  (re-exported)


def mamba2(heads, vdim, state, groups, conv, norm_groups):
    return dict(type="mamba2", mixer=dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups))


def attention(heads, kv_heads, dim, vdim, rot, base, scale=None, v_mix=False):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot=dict(dims=rot, base=base),
             scale=scale if scale is not None else 1.5 / math.sqrt(dim))
    if v_mix:
        m["v_mix"] = True
    return dict(type="attention", mixer=m)


def lightning(heads, dim, vdim, decay):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)))


def moe(experts, top, ff, limit):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


# Sizes that no matrix-core kernel takes (widths that are no multiple of 8, heads of 10, 8 and 12 with value heads of
# another size, a rotation of part of a head), an attention layer that mixes no values before the first that does, a
# layer without a feed-forward, several choices an expert, as many groups as heads and one group, two and four taps,
# decays of exactly 1 and 1/2, every layer of a kind with sizes of its own.
SMALL = dict(architecture="Tobozen", vocab=131, width=40, norm=dict(eps=1e-5, groups=4), layers=[
    layer(attention(3, 3, 10, 6, 4, 50.0, scale=0.4), moe(5, 2, 12, 0.5)),
    layer(lightning(3, 6, 10, [0.5, 0.875, 1.0]), None),
    layer(attention(4, 1, 8, 12, 8, 300.0, v_mix=True), moe(3, 3, 8, 7.0)),
    layer(mamba2(3, 5, 7, 3, 2, 3), moe(4, 1, 16, 1.5)),
    layer(attention(2, 2, 12, 6, 6, 10000.0, v_mix=True), None),
    layer(mamba2(4, 6, 4, 1, 4, 1), moe(6, 2, 4, 0.75)),
])
# Sizes that the matrix-core kernels take: attention heads of 64 and 32 whose values have the keys' size (whole and
# partial rotation), one of 128 with smaller values; states of 64 x 64, 16 x 32 and 128 x 64; every expert chosen; one
# norm group.
CORES = dict(architecture="Tobozen", vocab=520, width=256, norm=dict(eps=1e-6, groups=1), layers=[
    layer(mamba2(4, 64, 64, 1, 4, 4), moe(8, 2, 64, 2.0)),
    layer(attention(4, 1, 64, 64, 32, 100000.0, v_mix=True), moe(4, 4, 32, 1.0)),
    layer(lightning(2, 128, 64, [0.96875, 0.99609375]), None),
    layer(attention(8, 4, 32, 32, 32, 3000.0), moe(16, 3, 32, 3.0)),
    layer(attention(2, 2, 128, 32, 64, 1e6, v_mix=True), moe(8, 1, 96, 0.5)),
    layer(mamba2(8, 32, 16, 4, 3, 2), None),
    layer(lightning(4, 32, 96, [0.5, 0.75, 0.9375, 1.0]), moe(4, 2, 64, 1.0)),
])
CONFIGS = {"small": SMALL, "cores": CORES}
PAGE = {"small": 8, "cores": 16}
STORED = {"small": "F32", "cores": "BF16"}


def make_weights(cfg, seed):
    """name -> float32 array, every value a bfloat16 value (the engine in bf16 then holds what the plain
    implementation reads)."""
    rng = np.random.default_rng(seed)
    E, V = cfg["width"], cfg["vocab"]

    def n(shape, std, mean=0.0):
        return helpers.bf16_round(mean + rng.standard_normal(shape) * std)

    w = {"embed": n((V, E), 0.7), "final.norm": n(E, 0.1, 1.0)}
    for l, lc in enumerate(cfg["layers"]):
        p, m = f"l{l}.", lc["mixer"]
        w[p + "norm1"] = n(E, 0.1, 1.0)
        if lc["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, C = H * P, H * P + 2 * G * N
            w[p + "mix.in"] = n((2 * inner + 2 * G * N + H, E), 1.2 / math.sqrt(E))
            w[p + "mix.conv"] = n((C, m["conv"]), 0.5)
            w[p + "mix.conv.b"] = n(C, 0.1)
            w[p + "mix.dt_bias"] = n(H, 0.5, -0.5)
            w[p + "mix.A_log"] = n(H, 0.7, -1.5)
            w[p + "mix.D"] = n(H, 0.1, 1.0)
            w[p + "mix.norm"] = n(inner, 0.1, 1.0)
            w[p + "mix.o"] = n((E, inner), 0.7 / math.sqrt(inner))
        elif lc["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "mix.q"] = n((H * D, E), 1.0 / math.sqrt(E))
            w[p + "mix.k"] = n((G * D, E), 1.0 / math.sqrt(E))
            w[p + "mix.v"] = n((G * Dv, E), 1.0 / math.sqrt(E))
            w[p + "mix.q.norm"] = n(H * D, 0.1, 1.0)
            w[p + "mix.k.norm"] = n(G * D, 0.1, 1.0)
            if m.get("v_mix"):
                w[p + "mix.vmix"] = n((), 0.1, 0.4)
            w[p + "mix.o"] = n((E, H * Dv), 0.7 / math.sqrt(H * Dv))
        else:
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            for name, rows in (("q", H * D), ("k", H * D), ("v", H * Dv), ("g", H * Dv)):
                w[p + "mix." + name] = n((rows, E), 1.2 / math.sqrt(E))
            w[p + "mix.norm"] = n(H * Dv, 0.1, 1.0)
            w[p + "mix.o"] = n((E, H * Dv), 0.7 / math.sqrt(H * Dv))
        f = lc["mlp"]
        if f is None:
            continue
        w[p + "norm2"] = n(E, 0.1, 1.0)
        F = f["expert"]["ff"]
        w[p + "mlp.router"] = n((f["router"]["experts"], E), 2.0 / math.sqrt(E))
        for e in range(f["router"]["experts"]):
            w[f"{p}mlp.e{e}.gate"] = n((F, E), 1.5 / math.sqrt(E))
            w[f"{p}mlp.e{e}.up"] = n((F, E), 1.5 / math.sqrt(E))
            w[f"{p}mlp.e{e}.down"] = n((E, F), 1.0 / math.sqrt(F))
    return w


def make_model_dir(path, cfg, seed, weights=None, stored="F32"):
    """``stored``: F32 (a bf16 engine then keeps the matrices in 32-bit and runs the kernels for mixed operands) or
    BF16 (the kernels of the serving path)."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    helpers.write_safetensors(os.path.join(path, "model.safetensors"), weights if weights is not None else make_weights(cfg, seed), stored)
    return path


def random_requests(cfg, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab"], n)] for i, n in enumerate(lengths)}


def plain_logits(model_dir, reqs):
    cfg, w = pt.read_model(model_dir)
    return {r: pt.forward(cfg, w, toks) for r, toks in reqs.items()}


def forward_with_choices(cfg, w, tokens, chosen, margins=None):
    """The plain logits with the experts at (layer, position) taken from ``chosen`` ({(layer, position): ids}; the
    plain choice where it names none). ``margins`` receives {(layer, position): (the gap between the last chosen and
    the first not chosen plain score on that path, whether the given experts are the plain choice)}."""
    T = len(tokens)
    tops = {l: lc["mlp"]["router"]["top"] for l, lc in enumerate(cfg["layers"]) if lc["mlp"] is not None}
    choices = {}
    # a layer's scores depend on the choices of the layers before it: fix them layer by layer
    for l in sorted(tops):
        zs = {}
        pt.forward(cfg, w, tokens, choices=choices, router_out=zs)
        s = pt.sigmoid(zs[l])
        own, _ = pt.route(zs[l], tops[l])
        ids = own.copy()
        for t in range(T):
            forced = (chosen or {}).get((l, t))
            if forced is not None:
                ids[t] = forced
            if margins is not None:
                ordered = np.sort(s[t])[::-1]
                gap = ordered[tops[l] - 1] - ordered[tops[l]] if tops[l] < len(ordered) else np.inf
                margins[(l, t)] = (float(gap), set(int(e) for e in ids[t]) == set(int(e) for e in own[t]))
        choices[l] = ids
    return pt.forward(cfg, w, tokens, choices=choices)


def random_config(rng, big):
    """A configuration drawn at random: two to six layers of any kind in any order, with sizes that the matrix-core kernels
    take (``big``) or that none of them takes; layers that mix values agree on the values' width, as the design demands."""
    def pick(*xs):
        return xs[int(rng.integers(0, len(xs)))]
    width = pick(128, 256, 384) if big else pick(24, 40, 56, 72, 100)
    groups = pick(1, 2, 4)
    layers, mixed = [], None
    for _ in range(int(rng.integers(2, 7))):
        kind = pick("mamba2", "attention", "lightning")
        if kind == "mamba2":
            H = pick(2, 4, 6, 8)
            G = pick(*[g for g in (1, 2, 3, 4, 6, 8) if H % g == 0])
            P = pick(16, 32, 64, 40) if big else pick(4, 5, 12, 20)
            N = pick(16, 32, 48, 64, 128) if big else pick(3, 8, 17, 24)
            mix = mamba2(H, P, N, G, pick(1, 2, 3, 4), pick(*[g for g in (1, 2, 4, H) if (H * P) % g == 0]))
        elif kind == "attention":
            G = pick(1, 2, 4)
            H = G * pick(1, 2, 4, 7)
            D = pick(32, 64, 128) if big else pick(6, 10, 16, 24)
            v_mix = bool(rng.integers(0, 2))
            if v_mix and mixed is not None and mixed % G == 0:
                Dv = mixed // G
            elif v_mix and mixed is not None:
                v_mix, Dv = False, D
            else:
                Dv = pick(D, D // 2, 32 if big else 8)
            if v_mix and mixed is None:
                mixed = G * Dv
            rot = max(2, pick(D, D // 2, 2) // 2 * 2)
            mix = attention(H, G, D, Dv, rot, pick(100.0, 10000.0, 1e6), scale=pick(None, 0.2, 0.05), v_mix=v_mix)
        else:
            H = pick(1, 2, 3, 8)
            mix = lightning(H, pick(32, 64, 128) if big else pick(5, 8, 20), pick(32, 64, 96) if big else pick(4, 12, 30),
                            [pick(0.5, 0.75, 0.9375, 0.984375, 1.0) for _ in range(H)])
        E = pick(1, 2, 5, 8, 16)
        mlp = None if rng.random() < 0.25 else moe(E, int(rng.integers(1, min(E, 4) + 1)), pick(32, 64, 96, 48) if big else pick(4, 10, 24),
                                                   pick(0.5, 1.0, 3.0, 7.0))
        layers.append(layer(mix, mlp))
    return dict(architecture="Tobozen", vocab=int(rng.integers(50, 400)), width=width,
                norm=dict(eps=pick(1e-5, 1e-6), groups=groups if width % groups == 0 else 1), layers=layers)
