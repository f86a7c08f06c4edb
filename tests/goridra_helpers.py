"""Shared by the Goridra tests: small configurations that differ in every size and option, weights that make faults
visible, and the plain implementation's logits (optionally with the experts that the engine chose, see
``record_choices``)."""
import json
import math
import os

import numpy as np

import helpers
import plain_goridra as pg


def attention(heads, kv_heads, dim, vdim, rot, base, mask, scale=None, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot=dict(dims=rot, base=base), mask=dict(size=mask),
             scale=scale if scale is not None else 1.3 / math.sqrt(dim))
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, groups, keep, ff):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, groups=dict(count=groups, keep=keep)))


def layer(mixer, mlp):
    return dict(type="attention", mixer=mixer, mlp=mlp)


# Sizes that no matrix-core kernel takes (odd widths, a value head larger than the key head, a rotation of part of a
# head), a reader whose mask differs from its source's, a layer without a feed-forward, groups of which some are dropped.
SMALL = dict(architecture="Goridra", vocab=301, width=48, logit_softcap=9.0, norm=dict(eps=1e-5), layers=[
    layer(attention(4, 2, 12, 20, 8, 10000.0, 24), dense(72)),
    layer(attention(4, 2, 12, 20, 8, 10000.0, 16, scale=0.4, kv_from=0), moe(6, 2, 3, 2, 40)),
    layer(attention(3, 3, 16, 8, 16, 500.0, 40), None),
    layer(attention(6, 1, 8, 8, 2, 77.0, 7), moe(5, 1, 1, 1, 24)),
])
# Sizes that the matrix-core kernels take: heads of 64 and 32, whole and partial rotation, one group, every expert chosen.
CORES = dict(architecture="Goridra", vocab=520, width=256, logit_softcap=30.0, norm=dict(eps=1e-6), layers=[
    layer(attention(4, 1, 64, 64, 64, 100000.0, 48), dense(384)),
    layer(attention(4, 1, 64, 64, 64, 100000.0, 80, kv_from=0), moe(8, 1, 1, 1, 128)),
    layer(attention(8, 4, 32, 32, 16, 3000.0, 32), moe(4, 4, 4, 4, 64)),
    layer(attention(8, 4, 32, 32, 16, 3000.0, 32, kv_from=2), None),
    layer(attention(2, 2, 128, 128, 32, 1e6, 200), moe(16, 3, 4, 2, 32)),
])
CONFIGS = {"small": SMALL, "cores": CORES}
PAGE = {"small": 8, "cores": 16}
STORED = {"small": "F32", "cores": "BF16"}


def make_weights(cfg, seed):
    """name -> float32 array, every value a bfloat16 value (the engine in bf16 then holds what the plain
    implementation reads). Scales that give activations of order one and peaked attention."""
    rng = np.random.default_rng(seed)
    E, V = cfg["width"], cfg["vocab"]

    def n(shape, std):
        return helpers.bf16_round(rng.standard_normal(shape) * std)

    w = {"embed": n((V, E), 0.7), "final.norm": n(E, 0.1) + 1.0, "final.norm.b": n(E, 0.1)}
    for l, lc in enumerate(cfg["layers"]):
        p, m = f"l{l}.", lc["mixer"]
        w[p + "norm1"] = (1.0 + 0.1 * rng.standard_normal(E)).astype(np.float32)
        w[p + "norm1.b"] = (0.1 * rng.standard_normal(E)).astype(np.float32)
        w[p + "mix.q"] = n((m["heads"] * m["dim"], E), 1.2 / math.sqrt(E))
        if m.get("kv_from") is None:
            w[p + "mix.k"] = n((m["kv_heads"] * m["dim"], E), 1.2 / math.sqrt(E))
            w[p + "mix.v"] = n((m["kv_heads"] * m["vdim"], E), 1.0 / math.sqrt(E))
        w[p + "mix.o"] = n((E, m["heads"] * m["vdim"]), 0.7 / math.sqrt(m["heads"] * m["vdim"]))
        f = lc["mlp"]
        if f is None:
            continue
        if f["kind"] == "dense":
            w[p + "mlp.up"] = n((f["ff"], E), 1.0 / math.sqrt(E))
            w[p + "mlp.down"] = n((E, f["ff"]), 0.7 / math.sqrt(f["ff"]))
        else:
            F = f["expert"]["ff"]
            w[p + "mlp.router"] = n((f["router"]["experts"], E), 2.0 / math.sqrt(E))
            for e in range(f["router"]["experts"]):
                w[f"{p}mlp.e{e}.up"] = n((F, E), 1.0 / math.sqrt(E))
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


def plain_logits(model_dir, reqs, choices=None):
    """{request: logits [T, vocab]}. ``choices``: {request: {(layer, position): expert ids}} to take where given."""
    cfg, w = pg.read_model(model_dir)
    return {r: forward_with_choices(cfg, w, toks, (choices or {}).get(r)) for r, toks in reqs.items()}


def forward_with_choices(cfg, w, tokens, choices=None, margins=None):
    """``plain_goridra.forward`` with the router's choice replaced, at the places that ``choices`` names, by the given
    experts (their weights are still the plain scores over the sum of the chosen). ``margins``: a dict that receives
    {(layer, position): (the smallest gap between a score that decided the plain choice and the next one, whether the
    given experts are the plain choice)}, both for the scores on the path that the given choices lead along."""
    if not choices and margins is None:
        return pg.forward(cfg, w, tokens)
    original = pg.route
    state = {"layer": None}

    def route(z, top, n_groups, keep):
        ids, wts = original(z, top, n_groups, keep)
        s = pg.softmax(z)
        for t in range(z.shape[0]):
            forced = (choices or {}).get((state["layer"], t))
            if margins is not None:
                margins[(state["layer"], t)] = (choice_margin(s[t], top, n_groups, keep),
                                                forced is None or set(forced) == set(int(e) for e in ids[t]))
            if forced is not None:
                ids[t] = forced
                wts[t] = s[t, forced] / (s[t, forced].sum() + 1e-20)
        return ids, wts

    def moe_ff(h, router, ups, downs, top, n_groups, keep):
        state["layer"] = next(l for l in range(len(cfg["layers"])) if w.get(f"l{l}.mlp.router") is router)
        return original_moe(h, router, ups, downs, top, n_groups, keep)

    original_moe = pg.moe_ff
    pg.route, pg.moe_ff = route, moe_ff
    try:
        return pg.forward(cfg, w, tokens)
    finally:
        pg.route, pg.moe_ff = original, original_moe


def choice_margin(s, top, n_groups, keep):
    """How far the scores are from another choice: the gap at the border of the kept groups and at the border of the
    chosen experts (infinite where there is no border)."""
    E = len(s)
    per = E // n_groups
    gs = np.sort(s.reshape(n_groups, per).max(axis=1))[::-1]
    gap = gs[keep - 1] - gs[keep] if keep < n_groups else np.inf
    best = sorted(range(n_groups), key=lambda g: (-s.reshape(n_groups, per)[g].max(), g))[:keep]
    allowed = np.sort(np.concatenate([s[g * per:(g + 1) * per] for g in best]))[::-1]
    if top < len(allowed):
        gap = min(gap, allowed[top - 1] - allowed[top])
    return float(gap)


class record_choices:
    """While active, every mixture-of-experts layer of ``engine`` leaves the experts it chose:
    ``self.chosen[request][(layer, position)] = ids``. Steps must run eagerly (an engine made with ``graphs=False``)."""

    def __init__(self, engine):
        self.engine, self.chosen = engine, {}

    def __enter__(self):
        import torch
        from hf_cpu_amd.parts.moe import MixtureOfExperts
        self.cls, self.original = MixtureOfExperts, MixtureOfExperts.forward
        layer_of = {id(lay.named.get("feed_forward")): i for i, lay in enumerate(self.engine.model.layers)}
        outer = self

        def forward(part, ops, step, h, x):
            outer.original(part, ops, step, h, x)
            ids = ops.scratch("moe_ids", (h.shape[0], part.top), torch.int32).cpu().numpy()
            by_slot = {hd.slot: r for r, hd in outer.engine.manager.held.items()}
            for t, (pos, slot) in enumerate(zip(step.host["positions"], step.host["token_slot"])):
                if int(slot) in by_slot:
                    outer.chosen.setdefault(by_slot[int(slot)], {})[(layer_of[id(part)], int(pos))] = [int(e) for e in ids[t]]
        MixtureOfExperts.forward = forward
        return self

    def __exit__(self, *exc):
        self.cls.forward = self.original
        return False
