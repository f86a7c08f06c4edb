"""The plain implementation of the Tobozen design: whole sequences, float64 numpy, one function a mechanism.

No cache, no batching, no kernels, and no code shared with the package. The engine is compared with this.

A layer is ``x <- x + mixer(norm1(x))``, then ``x <- x + ff(norm2(x))`` where the layer has a feed-forward. The
norm divides each of ``groups`` equal runs of the vector by its own root mean square. Three mixers:

* ``mamba2``: a state-space layer. One projection gives a gate ``z``, inputs ``x``, ``B``, ``C`` and a step ``dt``;
  ``x | B | C`` pass a short causal convolution and silu; per head ``S <- exp(-exp(A) dt) S + dt B x^T`` and
  ``y = S^T C + D x``; ``y silu(z)`` is normed in groups and projected.
* ``attention``: grouped heads; queries and keys are normed over the whole projection, rotated in neighbouring pairs
  over the first ``rot.dims`` dimensions of a head; the softmax has one more term of score 0 and no value in its
  denominator; layers that mix values blend theirs with those of the first such layer.
* ``lightning``: linear attention with a fixed decay per head on silu'd queries, keys and values, normed, gated by a
  sigmoid and projected.

The feed-forward is a mixture of experts: sigmoid scores, the best ``top`` experts, the score scales the expert's
input, and an expert is a gated unit with clamped halves.
"""
import numpy as np

from plain import read_model          # the container reader is the same for every design


def group_rms_norm(x, w, eps, groups):
    """x: [..., n]. Each of ``groups`` equal consecutive runs is divided by sqrt(mean(run^2) + eps); then times w."""
    shape = x.shape
    g = x.reshape(shape[:-1] + (groups, shape[-1] // groups))
    g = g / np.sqrt((g * g).mean(axis=-1, keepdims=True) + eps)
    return g.reshape(shape) * w


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def causal_conv(u, taps, bias):
    """u: [T, C], taps: [C, K]. out[t, c] = bias[c] + sum_j taps[c, j] u[t - (K - 1) + j, c]; zeros before t = 0."""
    T, C = u.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), u], axis=0)
    out = np.tile(bias, (T, 1)).astype(np.float64)
    for j in range(K):
        out += padded[j:j + T] * taps[:, j]
    return out


def ssm_scan(x, B, C, dt, A_log, D):
    """x: [T, H, P], B and C: [T, G, N], dt: [T, H] (already positive). Head h reads group h // (H / G).
    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T  (S: [N, P]);  y_t = S_t^T C_t + D x_t."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    y = np.zeros((T, H, P))
    for h in range(H):
        g = h // (H // G)
        S = np.zeros((N, P))
        for t in range(T):
            S = np.exp(-np.exp(A_log[h]) * dt[t, h]) * S + dt[t, h] * np.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


def mamba2(h, w, p, m, eps):
    """The whole mixer on the normed stream h: [T, width]; w: tensors by name, p: their prefix, m: the mixer's sizes."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])
    y = ssm_scan(x, B, C, dt, w[p + "A_log"], w[p + "D"]).reshape(T, inner)
    y = group_rms_norm(y * silu(z), w[p + "norm"], eps, m["norm_groups"])
    return y @ w[p + "o"].T


def rotate_pairs(v, positions, dims, base):
    """v: [T, heads, dim]. Dimension 2i pairs with 2i + 1 for i < dims / 2; the pair (a, b) at position p becomes
    (a cos t - b sin t, b cos t + a sin t), t = p * base^(-2i/dims). Dimensions from ``dims`` on pass."""
    i = np.arange(dims // 2, dtype=np.float64)
    t = np.asarray(positions, dtype=np.float64)[:, None] * base ** (-2.0 * i / dims)
    c, s = np.cos(t)[:, None, :], np.sin(t)[:, None, :]
    out = v.copy()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def sink_softmax(s):
    """Rows of s (masked entries -inf): exp(s_j) / (1 + sum_j exp(s_j)), computed about the larger of max and 0."""
    m = np.maximum(s.max(axis=-1, keepdims=True), 0.0)
    e = np.exp(s - m)
    return e / (np.exp(-m) + e.sum(axis=-1, keepdims=True))


def attend(q, k, v, scale):
    """q: [T, H, D], k: [T, G, D], v: [T, G, Dv] -> [T, H * Dv]; causal; query head h reads head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    vis = np.arange(T)[None, :] <= np.arange(T)[:, None]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = np.where(vis, (q[:, h] @ k[:, g].T) * scale, -np.inf)
        out[:, h] = sink_softmax(s) @ v[:, g]
    return out.reshape(T, -1)


def attention(h, w, p, m, eps, positions, v_first):
    """Returns (output [T, width], the values this layer would hand on as the first layer's)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = group_rms_norm(h @ w[p + "q"].T, w[p + "q.norm"], eps, 1).reshape(T, H, D)
    k = group_rms_norm(h @ w[p + "k"].T, w[p + "k.norm"], eps, 1).reshape(T, G, D)
    v = h @ w[p + "v"].T
    q = rotate_pairs(q, positions, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_pairs(k, positions, m["rot"]["dims"], m["rot"]["base"])
    if m.get("v_mix") and v_first is not None:
        lam = float(w[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    return attend(q, k, v.reshape(T, G, Dv), m["scale"]) @ w[p + "o"].T, v


def lightning(h, w, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    k = silu(h @ w[p + "k"].T).reshape(T, H, D)
    v = silu(h @ w[p + "v"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        S = np.zeros((D, Dv))
        for t in range(T):
            S = m["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = group_rms_norm(o.reshape(T, H * Dv), w[p + "norm"], eps, 1) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def route(z, top):
    """z: [T, E] router logits -> (ids [T, top], weights [T, top]): the ``top`` largest sigmoid scores (the lower
    index among equals), and those scores as they are."""
    s = sigmoid(z)
    ids = np.stack([np.array(sorted(range(z.shape[1]), key=lambda e: (-s[t, e], e))[:top]) for t in range(z.shape[0])])
    return ids, np.take_along_axis(s, ids, axis=1)


def expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def moe_ff(h, w, p, f, choices=None):
    """``choices``: expert ids [T, top] to use instead of the router's own (their weights are still the scores)."""
    r = f["router"]
    z = h @ w[p + "router"].T
    ids, wts = route(z, r["top"])
    if choices is not None:
        ids = np.asarray(choices)
        wts = np.take_along_axis(sigmoid(z), ids, axis=1)
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], wts[t]):
            out[t] += expert(wt * h[t], w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"], f["expert"]["limit"])
    return out, z


def forward(cfg, w, tokens, layers_out=None, choices=None, router_out=None):
    """Logits [T, vocab] of one sequence from position 0. ``layers_out``: a list that receives the stream after every
    layer. ``choices``: {layer: ids [T, top]} to take the engine's experts; ``router_out``: a dict that receives each
    layer's router logits."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    T = len(tokens)
    pos = np.arange(T)
    x = w["embed"][np.asarray(tokens)].astype(np.float64)
    v_first = None
    for l, lc in enumerate(cfg["layers"]):
        p, m = f"l{l}.", lc["mixer"]
        h = group_rms_norm(x, w[p + "norm1"], eps, groups)
        if lc["type"] == "mamba2":
            x = x + mamba2(h, w, p + "mix.", m, eps)
        elif lc["type"] == "attention":
            y, v = attention(h, w, p + "mix.", m, eps, pos, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = v
            x = x + y
        elif lc["type"] == "lightning":
            x = x + lightning(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(lc["type"])
        f = lc.get("mlp")
        if f is not None:
            h = group_rms_norm(x, w[p + "norm2"], eps, groups)
            y, z = moe_ff(h, w, p + "mlp.", f, None if choices is None else choices.get(l))
            if router_out is not None:
                router_out[l] = z
            x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    x = group_rms_norm(x, w["final.norm"], eps, groups)
    return x @ w["embed"].T


__all__ = ["read_model", "group_rms_norm", "silu", "sigmoid", "softplus", "causal_conv", "ssm_scan", "mamba2",
           "rotate_pairs", "sink_softmax", "attend", "attention", "lightning", "route", "expert", "moe_ff", "forward"]
