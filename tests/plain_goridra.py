"""The plain implementation of the Goridra design: whole sequences, float64 numpy, one function a mechanism.

No cache, no batching, no kernels, and no code shared with the package. The engine is compared with this.

A layer is ``x <- x + mixer(h) + ff(h)`` with ``h = layer_norm(x)``: both branches read one norm. The mixer
is softmax attention with grouped heads, a rotation of the first ``rot.dims`` dimensions of each query and key
head, and a mask by chunks: a query at ``i`` sees the keys ``j <= i`` of its own chunk, ``i // size == j // size``.
A layer whose mixer names ``kv_from`` has no keys and values of its own and uses that layer's. The feed-forward is
dense (erf gelu) or a mixture of experts (softmax router, best groups, best experts, squared relu). The logits are
the tied embedding's products, squashed by ``cap * tanh(. / cap)``.
"""
import math

import numpy as np

from plain import read_model, softmax          # the container reader and the row softmax are the same for every design

_erf = np.vectorize(math.erf, otypes=[np.float64])


def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b over the last axis; var is the mean squared deviation."""
    mu = x.mean(axis=-1, keepdims=True)
    d = x - mu
    var = (d * d).mean(axis=-1, keepdims=True)
    return d / np.sqrt(var + eps) * w + b


def rotate(v, positions, dims, base):
    """v: [T, heads, dim]. Dimension i < dims/2 pairs with i + dims/2; the pair (a, b) at position p becomes
    (a cos t - b sin t, b cos t + a sin t), t = p * base^(-2i/dims). Dimensions from ``dims`` on pass."""
    half = dims // 2
    i = np.arange(half, dtype=np.float64)
    t = np.asarray(positions, dtype=np.float64)[:, None] * base ** (-2.0 * i / dims)
    c, s = np.cos(t)[:, None, :], np.sin(t)[:, None, :]
    out = v.copy()
    a, b = v[..., :half], v[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def chunk_visible(n, size):
    """[n, n] booleans: query i sees key j iff j <= i and both lie in one chunk of ``size`` positions."""
    i = np.arange(n)[:, None]
    j = np.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def attend(q, k, v, scale, size):
    """q: [T, H, D], k: [T, G, D], v: [T, G, Dv] -> [T, H * Dv]; query head h reads key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    vis = chunk_visible(T, size)
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(vis, s, -np.inf)
        out[:, h] = softmax(s) @ v[:, g]
    return out.reshape(T, -1)


def gelu_erf(z):
    return 0.5 * z * (1.0 + _erf(z / math.sqrt(2.0)))


def dense_ff(h, up, down):
    return gelu_erf(h @ up.T) @ down.T


def route(z, top, n_groups, keep):
    """z: [T, E] router logits -> (ids [T, top], weights [T, top]). Scores are the softmax over all experts; a group
    of neighbours scores as its best expert; the ``top`` best experts of the ``keep`` best groups are chosen and
    weigh as their scores over the sum of the chosen scores."""
    T, E = z.shape
    s = softmax(z)
    per = E // n_groups
    gs = s.reshape(T, n_groups, per).max(axis=2)
    ids = np.zeros((T, top), dtype=np.int64)
    wts = np.zeros((T, top))
    for t in range(T):
        best = sorted(range(n_groups), key=lambda g: (-gs[t, g], g))[:keep]
        allowed = [e for e in range(E) if e // per in best]
        chosen = sorted(allowed, key=lambda e: (-s[t, e], e))[:top]
        ids[t] = chosen
        wts[t] = s[t, chosen] / (s[t, chosen].sum() + 1e-20)
    return ids, wts


def moe_ff(h, router, ups, downs, top, n_groups, keep):
    ids, wts = route(h @ router.T, top, n_groups, keep)
    out = np.zeros((h.shape[0], downs[0].shape[0]))
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], wts[t]):
            a = np.maximum(h[t] @ ups[e].T, 0.0) ** 2
            out[t] += wt * (a @ downs[e].T)
    return out


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence from position 0. ``layers_out``: a list that receives the stream after
    every layer."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    pos = np.arange(T)
    x = w["embed"][np.asarray(tokens)]
    kv = {}
    for l, lc in enumerate(cfg["layers"]):
        p, m = f"l{l}.", lc["mixer"]
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = rotate((h @ w[p + "mix.q"].T).reshape(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"])
        if m.get("kv_from") is None:
            k = rotate((h @ w[p + "mix.k"].T).reshape(T, G, D), pos, m["rot"]["dims"], m["rot"]["base"])
            kv[l] = (k, (h @ w[p + "mix.v"].T).reshape(T, G, Dv))
        k, v = kv[l if m.get("kv_from") is None else m["kv_from"]]
        y = attend(q, k, v, m["scale"], m["mask"]["size"]) @ w[p + "mix.o"].T
        f = lc.get("mlp")
        if f is not None:
            if f["kind"] == "dense":
                y = y + dense_ff(h, w[p + "mlp.up"], w[p + "mlp.down"])
            else:
                r = f["router"]
                ups = [w[f"{p}mlp.e{e}.up"] for e in range(r["experts"])]
                downs = [w[f"{p}mlp.e{e}.down"] for e in range(r["experts"])]
                y = y + moe_ff(h, w[p + "mlp.router"], ups, downs, r["top"], r["groups"]["count"], r["groups"]["keep"])
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    logits = x @ w["embed"].T
    cap = cfg["logit_softcap"]
    return cap * np.tanh(logits / cap)


__all__ = ["read_model", "layer_norm", "rotate", "chunk_visible", "attend", "gelu_erf", "dense_ff", "route", "moe_ff",
           "forward"]
