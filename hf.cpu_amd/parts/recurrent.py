"""Mixers that keep per-request state of fixed size instead of a growing cache: a state-space layer and linear
attention with a fixed decay. Both walk a request's tokens in order from the state the step before left, with one
kernel for the recurrence (``Ops.linear_scan``): ``S <- a_t S + k_t (b_t v_t)^T``, ``y_t = S^T q_t + d v_t``."""
import torch

from .. import memory
from ..kernels.ops import Ops
from ..registry import register_part
from ..status import EINVAL, fail
from .base import FixedState, ParamSpec, Part


@register_part("mixer", "mamba2")
class Mamba2(Part):
    """A state-space layer with a scalar decay per head and step. With ``inner = n_heads * head_dim``, N = ``state_size``
    and G = ``n_groups``, one projection of the input gives ``[z: inner | x: inner | B: G N | C: G N | dt: n_heads]``.
    ``x | B | C`` pass a causal convolution per channel over ``conv_taps`` inputs (the last tap is the current token's;
    zeros before a sequence's start) with a bias, and silu. ``dt <- softplus(dt + dt_bias)``. Per head h, with B and C of
    group ``h // (n_heads / G)``: ``S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T`` (S: N x head_dim),
    ``y_t = S_t^T C_t + D_h x_t``. Then ``y silu(z)`` is RMS-normed in ``norm_groups`` equal runs (weight ``norm``) and
    projected: ``x += Wo (...)``.

    Decays, step sizes, the recurrence and the norm are fp32; the state (S of every head, and the convolution's last
    ``conv_taps - 1`` inputs) is fp32 in the request's state row. ``names``: the tensors' names after ``prefix`` (keys
    in, conv, conv_bias, dt_bias, a_log, d, norm, o)."""
    graph_safe = True

    def __init__(self, hidden_size, n_heads, head_dim, state_size, n_groups, conv_taps, norm_groups, eps, prefix="", names=None):
        super().__init__(prefix)
        if n_heads % n_groups:
            fail(EINVAL, f"mamba2: {n_heads} heads are not a multiple of {n_groups} groups")
        self.E, self.H, self.P, self.N, self.G, self.K = hidden_size, n_heads, head_dim, state_size, n_groups, conv_taps
        self.inner = n_heads * head_dim
        if norm_groups <= 0 or self.inner % norm_groups:
            fail(EINVAL, f"mamba2: {self.inner} inner values do not form {norm_groups} equal runs")
        self.norm_groups, self.eps = norm_groups, float(eps)
        self.C = self.inner + 2 * n_groups * state_size            # channels of the convolution
        self.W_in = 2 * self.inner + 2 * n_groups * state_size + n_heads
        self.n_scan = Ops.scan_state_floats(n_heads, state_size, head_dim)    # of the recurrence in a state row; the convolution's follow
        self.names = {"in": "in_proj.weight", "conv": "conv.weight", "conv_bias": "conv.bias", "dt_bias": "dt_bias",
                      "a_log": "A_log", "d": "D", "norm": "norm.weight", "o": "out_proj.weight"}
        self.names.update(names or {})
        self.w_in = self.taps = self.conv_bias = self.dt_bias = self.a_log = self.d = self.norm_w = self.w_o = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        return [ParamSpec(p + nm["in"], (self.W_in, self.E)),
                ParamSpec(p + nm["conv"], (self.C, self.K), "vector", ("normal", 0.3)),
                ParamSpec(p + nm["conv_bias"], (self.C,), "vector", ("normal", 0.1)),
                ParamSpec(p + nm["dt_bias"], (self.H,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["a_log"], (self.H,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["d"], (self.H,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["norm"], (self.inner,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["o"], (self.E, self.inner))]

    def cache_need(self):
        return FixedState(self.n_scan + (self.K - 1) * self.C)

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        self.w_in, self.w_o = params[p + nm["in"]], params[p + nm["o"]]
        self.taps, self.conv_bias = params[p + nm["conv"]].contiguous(), params[p + nm["conv_bias"]]
        self.dt_bias, self.a_log, self.d = params[p + nm["dt_bias"]], params[p + nm["a_log"]], params[p + nm["d"]]
        self.norm_w = params[p + nm["norm"]]

    def forward(self, ops, step, h, cache, x, write_cache=True):
        if not write_cache:
            fail(EINVAL, f"mamba2 '{self.prefix}': a state cannot be read without being advanced")
        T, inner, GN = h.shape[0], self.inner, self.G * self.N
        proj = ops.scratch("ssm_in", (T, self.W_in), ops.act_dtype)
        with ops.section("ssm_in"):
            ops.gemm(h, self.w_in, proj)
        xbc = ops.scratch("ssm_conv", (T, self.C), torch.float32)
        y = ops.scratch("ssm_y", (T, inner), torch.float32)
        with ops.section("ssm_conv"):
            ops.causal_conv(proj[:, inner:inner + self.C], self.taps, self.conv_bias, cache.state[:, self.n_scan:], step, xbc,
                            activation="silu")
        with ops.section("ssm_scan"):
            ops.linear_scan(xbc[:, inner + GN:], xbc[:, inner:inner + GN], xbc[:, :inner], self.G, self.N, self.H, self.P,
                            cache.state, step, y, step_size=proj[:, inner + self.C:], step_bias=self.dt_bias, a_log=self.a_log,
                            skip=self.d)
        gated = ops.scratch("ssm_gated", (T, inner), ops.act_dtype)
        with ops.section("ssm_norm"):
            ops.group_rmsnorm(y, self.norm_w, self.eps, self.norm_groups, gated, gate=proj[:, :inner], gate_kind="silu_before")
        with ops.section("ssm_wo"):
            ops.gemm(gated, self.w_o, x, accumulate=True, defer=True)


@register_part("mixer", "lightning")
class LightningAttention(Part):
    """Linear attention with a fixed decay per head: ``q = silu(Wq h)``, ``k = silu(Wk h)`` (``n_heads`` x ``head_dim``),
    ``v = silu(Wv h)`` (``n_heads`` x ``v_head_dim``); per head ``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``,
    no other scale. The heads together are RMS-normed (weight ``norm``), multiplied by ``sigmoid(Wg h)`` and projected:
    ``x += Wo (...)``. The state is fp32 in the request's state row, as are the recurrence and the norm. ``names``: the
    tensors' names after ``prefix`` (keys q, k, v, g, norm, o)."""
    graph_safe = True

    def __init__(self, hidden_size, n_heads, head_dim, v_head_dim, decay, eps, prefix="", names=None):
        super().__init__(prefix)
        decay = tuple(float(d) for d in decay)
        if len(decay) != n_heads or not all(0.0 <= d <= 1.0 for d in decay):
            fail(EINVAL, f"lightning: {n_heads} heads need as many decays between 0 and 1, got {len(decay)}")
        self.E, self.H, self.D, self.Dv = hidden_size, n_heads, head_dim, v_head_dim
        self.decay_values, self.eps = decay, float(eps)
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight",
                      "norm": "norm.weight", "o": "out_proj.weight"}
        self.names.update(names or {})
        self.w_qkv = self.w_g = self.w_o = self.norm_w = self.decay = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        QD, VD = self.H * self.D, self.H * self.Dv
        return [ParamSpec(p + nm["q"], (QD, self.E)), ParamSpec(p + nm["k"], (QD, self.E)), ParamSpec(p + nm["v"], (VD, self.E)),
                ParamSpec(p + nm["g"], (VD, self.E)), ParamSpec(p + nm["norm"], (VD,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["o"], (self.E, VD))]

    def cache_need(self):
        return FixedState(Ops.scan_state_floats(self.H, self.D, self.Dv))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm[n]] for n in "qkv"]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k and v in one matrix")
        self.w_g, self.w_o, self.norm_w = params[p + nm["g"]], params[p + nm["o"]], params[p + nm["norm"]]
        self.decay = memory.to_device(torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32), ops.device,
                                      f"{p}decays")

    def forward(self, ops, step, h, cache, x, write_cache=True):
        if not write_cache:
            fail(EINVAL, f"lightning '{self.prefix}': a state cannot be read without being advanced")
        T, QD, VD = h.shape[0], self.H * self.D, self.H * self.Dv
        qkv = ops.scratch("lin_qkv", (T, 2 * QD + VD), ops.act_dtype)
        gate = ops.scratch("lin_gate", (T, VD), ops.act_dtype)
        with ops.section("lin_qkv"):
            ops.gemm(h, self.w_qkv, qkv, activation="silu")
            ops.gemm(h, self.w_g, gate)
        o = ops.scratch("lin_o", (T, VD), torch.float32)
        with ops.section("lin_scan"):
            ops.linear_scan(qkv[:, :QD], qkv[:, QD:2 * QD], qkv[:, 2 * QD:], self.H, self.D, self.H, self.Dv, cache.state, step, o,
                            decay=self.decay)
        normed = ops.scratch("lin_normed", (T, VD), ops.act_dtype)
        with ops.section("lin_norm"):
            ops.group_rmsnorm(o, self.norm_w, self.eps, 1, normed, gate=gate, gate_kind="sigmoid_after")
        with ops.section("lin_wo"):
            ops.gemm(normed, self.w_o, x, accumulate=True, defer=True)
