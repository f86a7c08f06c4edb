"""Tobozen as a plan: pre-norm layers (RMS norms in groups) whose mixer is, layer by layer, a state-space layer, softmax
attention (queries and keys normed whole, rotated in neighbouring pairs, one more term of score 0 in the softmax, values
blended with the first such layer's) or linear attention with a fixed decay, followed by a mixture of gated experts whose
weights scale their inputs; logits from the tied embedding.

Tensor names: ``embed``; ``l<i>.norm1``, ``l<i>.norm2``; ``l<i>.mix.*`` (``in``, ``conv``, ``conv.b``, ``dt_bias``, ``A_log``,
``D``, ``norm``, ``o`` / ``q``, ``k``, ``v``, ``q.norm``, ``k.norm``, ``vmix``, ``o`` / ``q``, ``k``, ``v``, ``g``, ``norm``, ``o``);
``l<i>.mlp.router`` and ``l<i>.mlp.e<n>.{gate,up,down}``; ``final.norm``.
"""
from ..config.tobozen import TobozenConfig
from ..plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..registry import register_architecture

EXPERT_ALPHA = 1.702          # an expert's gate half is g sigmoid(1.702 g)
EXPERT_SHIFT = 1.0            # and its up half enters as u + 1


def _norm(cfg, name, optional=False):
    return PartSpec("group_rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps, groups=cfg.norm_groups, weight="", prefix=name,
                                          optional=optional))


def tobozen_plan(cfg):
    E = cfg.width
    layers, schedule = [], []
    first_mix_seen = False
    for l, lc in enumerate(cfg.layers):
        prefix, m = f"l{l}.", lc.mixer
        if lc.type == "mamba2":
            mixer = PartSpec("mamba2", dict(
                hidden_size=E, n_heads=m.heads, head_dim=m.vdim, state_size=m.state, n_groups=m.groups, conv_taps=m.conv,
                norm_groups=m.norm_groups, eps=cfg.norm_eps, prefix=prefix + "mix.",
                names={"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
                       "norm": "norm", "o": "o"}))
        elif lc.type == "attention":
            rotary = PartSpec("rotary", dict(head_dim=m.dim, rot_dim=m.rot_dims, theta=m.rot_base, pairing="interleaved"))
            v_mix = None
            if m.v_mix:
                v_mix = "blend" if first_mix_seen else "first"
                first_mix_seen = True
            mixer = PartSpec("attention", dict(
                hidden_size=E, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_head_dim=m.vdim, qkv_bias=False,
                window=0, scale=m.scale, position=rotary, qk_norm=cfg.norm_eps, sink=True, v_mix=v_mix,
                names=dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm", v_mix="vmix"), prefix=prefix + "mix."))
        else:
            mixer = PartSpec("lightning", dict(
                hidden_size=E, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, decay=m.decay, eps=cfg.norm_eps,
                prefix=prefix + "mix.", names=dict(q="q", k="k", v="v", g="g", norm="norm", o="o")))
        parts = dict(norm1=_norm(cfg, prefix + "norm1"), mixer=mixer)
        f = lc.mlp
        if f is None:
            parts["norm2"] = _norm(cfg, prefix + "norm2", optional=True)      # never run; a file may hold its weight all the same
        else:
            parts["norm2"] = _norm(cfg, prefix + "norm2")
            parts["feed_forward"] = PartSpec("moe", dict(
                hidden_size=E, expert_size=f.ff, n_experts=f.experts, top=f.top, n_groups=1, keep_groups=1, scoring="sigmoid",
                renormalize=False, weight_on="input", gated=dict(alpha=EXPERT_ALPHA, limit=f.limit, shift=EXPERT_SHIFT),
                names=dict(router="router", gate="e{e}.gate", up="e{e}.up", down="e{e}.down"), prefix=prefix + "mlp."))
        layers.append(LayerPlan.of(prefix, PartSpec("prenorm", dict(hidden_size=E)), **parts))
        schedule.append(ScheduleEntry(l))
    return ModelPlan(
        hidden_size=E, vocab_size=cfg.vocab,
        embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab, hidden_size=E, prefix="", weight="embed")),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=E, tied=True, tied_to="embed", prefix="head.")),
    ).check()


register_architecture("Tobozen", TobozenConfig, tobozen_plan)
