"""Softmax attention over a paged key/value cache, with grouped heads and an
optional window."""
import math

import torch

from .. import memory

from ..registry import make_part, register_part
from ..status import EINVAL, fail
from .base import PagedKV, ParamSpec, Part


@register_part("mixer", "attention")
class Attention(Part):
    """``q = Wq h + bq`` etc. (src/model.c:581-585); position encoding on q and k;
    for query head ``h`` the key/value head is ``h / (heads / kv_heads)``; scores
    ``dot(q, k) * scale`` over the visible keys, softmax in fp32, weighted sum of
    values (src/model.c:499-528); ``x += Wo att`` (src/model.c:606-609).

    A key at ``pk`` is visible to a query at ``pq`` iff ``0 <= pq - pk`` and, when
    ``window > 0``, ``pq - pk < window``, and, when ``mask_chunk > 0``, ``pq // mask_chunk == pk // mask_chunk``
    (runs of ``mask_chunk`` positions counted from the start of the sequence, wherever a prompt was cut).

    ``own_kv=False``: the mixer has no key and value projections and no cache of its own; the plan's schedule lets
    its entry read an earlier entry's cache (``ScheduleEntry.cache_of``), with its own queries, scale and mask.

    ``names`` gives the tensors' names after ``prefix`` (keys q, k, v, o, and q_bias, k_bias, v_bias, o_bias).

    A position encoding that enters the scores instead of the queries and keys has an
    attribute ``score_slopes`` (fp32 on the device, one per query head): the score then is
    ``dot(q, k) * scale + score_slopes[h] * (pk - pq)``.

    ``qk_norm`` = eps: queries and keys are RMS-normed over the whole projection (all heads at once) with the weights
    ``q_norm`` and ``k_norm`` (names in ``names``), before the rotation. ``sink``: the softmax has one more term of score 0
    that has no value, ``p_j = exp(s_j) / (1 + sum exp(s_i))``. ``v_mix``: ``"first"``: this layer's values, as projected,
    are kept for the step; ``"blend"``: ``v <- (1 - l) v + l v_first`` with the scalar tensor ``v_mix`` (name in
    ``names``) and the kept values of the same token; the blended values are what is cached. A ``"first"`` layer holds the
    scalar too, unused.
    """
    graph_safe = True
    lazy_input_ok = True


    def __init__(self, hidden_size, n_heads, n_kv_heads, head_dim, qkv_bias, window, position,
                 scale=None, out_bias=False, v_head_dim=None, prefix="", mask_chunk=0, own_kv=True, names=None,
                 qk_norm=None, sink=False, v_mix=None):
        """``v_head_dim``: the size of a value head where it is not ``head_dim`` (key rows of the cache are
        then ``n_kv_heads * head_dim`` wide, value rows ``n_kv_heads * v_head_dim``, and the output
        projection reads ``n_heads * v_head_dim`` columns; such a mixer runs the plain kernels)."""
        super().__init__(prefix)
        if n_heads % n_kv_heads:
            fail(EINVAL, f"attention: {n_heads} heads are not a multiple of {n_kv_heads} key/value heads")
        self.E, self.H, self.G, self.D = hidden_size, n_heads, n_kv_heads, head_dim
        self.Dv = head_dim if v_head_dim is None else int(v_head_dim)
        self.QD, self.KD = n_heads * head_dim, n_kv_heads * head_dim
        self.VD, self.OD = n_kv_heads * self.Dv, n_heads * self.Dv
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = int(window)
        self.mask_chunk = int(mask_chunk)
        self.own_kv = bool(own_kv)
        self.names = {n: f"{n}_proj.weight" for n in "qkvo"}
        self.names.update({f"{n}_bias": f"{n}_proj.bias" for n in "qkvo"})
        self.names.update(q_norm="q_norm.weight", k_norm="k_norm.weight", v_mix="v_mix")
        self.names.update(names or {})
        self.qk_norm = None if qk_norm is None else float(qk_norm)
        self.sink = bool(sink)
        if v_mix not in (None, "first", "blend") or (v_mix and not own_kv):
            fail(EINVAL, f"attention: v_mix '{v_mix}' is neither first nor blend, or the layer has no values of its own")
        self.v_mix = v_mix
        self.q_norm_w = self.k_norm_w = self.v_blend = None
        if self.window < 0 or self.mask_chunk < 0:
            fail(EINVAL, "attention: a window and a masking chunk are counted in tokens, 0 for none")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # src/model.c:507
        self.position = make_part("position", position)
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    def sub_parts(self):
        return [self.position]

    def param_specs(self):
        p, nm = self.prefix, self.names
        widths = {"q": self.QD, "k": self.KD, "v": self.VD}
        specs = [ParamSpec(p + nm[n], (widths[n], self.E)) for n in self._projections()]
        specs.append(ParamSpec(p + nm["o"], (self.E, self.OD)))
        if self.qkv_bias:
            specs += [ParamSpec(p + nm[n + "_bias"], (widths[n],), "vector") for n in self._projections()]
        if self.out_bias:
            specs.append(ParamSpec(p + nm["o_bias"], (self.E,), "vector"))
        if self.qk_norm is not None:
            specs.append(ParamSpec(p + nm["q_norm"], (self.QD,), "vector", ("one_plus_normal", 0.1)))
            if self.own_kv:
                specs.append(ParamSpec(p + nm["k_norm"], (self.KD,), "vector", ("one_plus_normal", 0.1)))
        if self.v_mix:
            specs.append(ParamSpec(p + nm["v_mix"], (), "vector", ("normal", 0.3), optional=self.v_mix == "first"))
        return specs

    def _projections(self):
        return "qkv" if self.own_kv else "q"

    def cache_need(self):
        if not self.own_kv:
            fail(EINVAL, f"attention '{self.prefix}' has no keys and values of its own: its schedule entry must read "
                         "another entry's cache")
        return PagedKV(self.KD, self.VD, self.window, self.mask_chunk)

    def reads_cache(self, need):
        """``need`` of the mixer whose storage this one reads, widened by what this one sees of it."""
        return PagedKV(need.k_width, need.v_width, need.window, need.mask_chunk, need.readers + ((self.window, self.mask_chunk),))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        # One matrix for the three projections that share an input: rows of q, then k, then v.
        mats = [params[p + nm[n]] for n in self._projections()]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k and v in one matrix")
        if self.qkv_bias:
            self.b_qkv = memory.cat([params[p + nm[n + "_bias"]] for n in self._projections()], 0,
                                    f"{p}q, k and v biases in one vector")
        self.w_o = params[p + nm["o"]]
        self.short_request_rows = ops.prompt_rows     # where the attention kernels for decoded tokens and for prompt portions part
        if self.out_bias:
            self.b_o = params[p + nm["o_bias"]]
        if self.qk_norm is not None:
            self.q_norm_w = params[p + nm["q_norm"]]
            self.k_norm_w = params[p + nm["k_norm"]] if self.own_kv else None
        if self.v_mix == "blend":
            self.v_blend = params[p + nm["v_mix"]].reshape(1)

    def forward(self, ops, step, h, cache, x, write_cache=True):
        T = h.shape[0]
        if write_cache and not self.own_kv:
            fail(EINVAL, f"attention '{self.prefix}' has no keys and values to write")
        width = self.QD + self.KD + self.VD if write_cache else self.QD
        qkv = ops.scratch("qkv", (T, width), ops.act_dtype)
        # a product that split K is added up inside the next kernel (position.store, the next norm)
        with ops.section("qkv"):
            ops.gemm(h, self.w_qkv[:width], qkv, bias=None if self.b_qkv is None else self.b_qkv[:width], defer=True)
        prepare = {}
        if self.qk_norm is not None:
            prepare.update(q_norm=self.q_norm_w, k_norm=self.k_norm_w if write_cache else None, eps=self.qk_norm)
        if self.v_mix and write_cache:
            # the first mixing layer's values of this step's tokens wait in a work buffer for the layers that blend
            kept = ops.scratch("v_first", (T, self.VD), ops.act_dtype)
            prepare.update(dict(v_keep=kept) if self.v_mix == "first" else dict(v_blend=self.v_blend, v_other=kept))
        if prepare:
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache, v_head_dim=self.Dv,
                                prepare=prepare)
        elif self.Dv == self.D:
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache)
        else:                                   # only a position part that knows of value heads of another size can serve
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache, v_head_dim=self.Dv)
        att = ops.scratch("att", (T, self.OD), ops.act_dtype)
        with ops.section("attn"):
            ops.paged_attention(qkv, self.H, self.G, self.D, cache, step, self.window, self.scale, att,
                                slopes=getattr(self.position, "score_slopes", None), v_head_dim=self.Dv,
                                mask_chunk=self.mask_chunk, sink=self.sink)
        with ops.section("wo"):
            ops.gemm(att, self.w_o, x, bias=self.b_o, accumulate=True, defer=True)
