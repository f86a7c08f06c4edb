"""Goridra as a plan: parallel layers (one layer norm, attention and feed-forward side by side), attention masked by
chunks with partly rotated heads, layers that read an earlier layer's keys and values, dense or mixture-of-experts
feed-forwards, and soft-capped logits from the tied embedding.

Tensor names: ``embed``; ``l<i>.norm1`` and ``l<i>.norm1.b``; ``l<i>.mix.{q,k,v,o}`` (no k and v where the layer reads
another's); ``l<i>.mlp.{up,down}`` or ``l<i>.mlp.router`` and ``l<i>.mlp.e<n>.{up,down}``; ``final.norm`` and ``final.norm.b``.
"""
from ..config.goridra import GoridraConfig
from ..plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..registry import register_architecture


def goridra_plan(cfg):
    E = cfg.width
    layers, schedule = [], []
    for l, lc in enumerate(cfg.layers):
        prefix, m = f"l{l}.", lc.mixer
        rotary = PartSpec("rotary", dict(head_dim=m.dim, rot_dim=m.rot_dims, theta=m.rot_base))
        parts = dict(
            norm1=PartSpec("layernorm", dict(size=E, eps=cfg.norm_eps, weight="", bias=".b", prefix=prefix + "norm1")),
            mixer=PartSpec("attention", dict(
                hidden_size=E, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_head_dim=m.vdim, qkv_bias=False,
                window=0, mask_chunk=m.mask_size, scale=m.scale, position=rotary, own_kv=m.kv_from is None,
                names=dict(q="q", k="k", v="v", o="o"), prefix=prefix + "mix.")))
        f = lc.mlp
        if f is not None and f.kind == "dense":
            parts["feed_forward"] = PartSpec("mlp", dict(hidden_size=E, intermediate_size=f.ff, activation="gelu_erf",
                                                         names=dict(up="up", down="down"), prefix=prefix + "mlp."))
        elif f is not None:
            parts["feed_forward"] = PartSpec("moe", dict(
                hidden_size=E, expert_size=f.ff, n_experts=f.experts, top=f.top, n_groups=f.groups, keep_groups=f.keep,
                activation="relu2", scoring="softmax", renormalize=True,
                names=dict(router="router", up="e{e}.up", down="e{e}.down"), prefix=prefix + "mlp."))
        layers.append(LayerPlan.of(prefix, PartSpec("parallel", dict(hidden_size=E)), **parts))
        schedule.append(ScheduleEntry(l, m.kv_from))
    return ModelPlan(
        hidden_size=E, vocab_size=cfg.vocab,
        embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab, hidden_size=E, prefix="", weight="embed")),
        layers=tuple(layers), schedule=tuple(schedule),
        final_norm=PartSpec("layernorm", dict(size=E, eps=cfg.norm_eps, weight="", bias=".b", prefix="final.norm")),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=E, tied=True, tied_to="embed", prefix="head.",
                                     softcap=cfg.logit_softcap)),
    ).check()


register_architecture("Goridra", GoridraConfig, goridra_plan)
