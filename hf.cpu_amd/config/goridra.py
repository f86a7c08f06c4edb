"""The typed configuration of the Goridra design.

config.json: ``architecture`` (the name), ``vocab``, ``width``, ``logit_softcap``, ``norm.eps`` and ``layers``, a list with
one object a layer: ``type`` (the kind of mixer: ``attention``), ``mixer`` (``heads``, ``kv_heads``, ``dim``, ``vdim``,
``scale``, ``rot.dims``, ``rot.base``, ``mask.size`` and, for a layer that reads another layer's keys and values,
``kv_from``) and ``mlp`` (null, or ``kind`` ``dense`` with ``ff``, or ``kind`` ``moe`` with ``expert.ff`` and
``router.experts``, ``router.top``, ``router.groups.count``, ``router.groups.keep``). Every size and constant of a
model comes from there; layers may differ from one another in all of them.
"""
from dataclasses import dataclass
from typing import Optional

from ..status import EFORMAT, ENOTSUP, fail
from .reader import KeyReader


@dataclass(frozen=True)
class GoridraAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    mask_size: int
    kv_from: Optional[int]


@dataclass(frozen=True)
class GoridraMLP:
    kind: str                    # "dense" or "moe"
    ff: int                      # of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1


@dataclass(frozen=True)
class GoridraLayer:
    type: str
    mixer: GoridraAttention
    mlp: Optional[GoridraMLP]


@dataclass(frozen=True, eq=False)
class GoridraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    logit_softcap: float
    layers: tuple
    raw: dict                    # config.json as read (to_dict gives it back)

    @staticmethod
    def _sub(r, key):
        v = r.obj.get(key)
        if not isinstance(v, dict):
            fail(EFORMAT, f"{r.origin}: key '{key}' is missing or not an object")
        return KeyReader(v, f"{r.origin}: {key}")

    @classmethod
    def from_dict(cls, obj, origin="config.json"):
        r = KeyReader(obj, origin)
        raw_layers = obj.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            fail(EFORMAT, f"{origin}: key 'layers' is missing or not a list of layers")
        layers = []
        for i, lo in enumerate(raw_layers):
            lr = KeyReader(lo, f"{origin}: layers[{i}]")
            kind = lr.string("type")
            if kind != "attention":
                fail(ENOTSUP, f"{lr.origin}: a mixer of type '{kind}' is not supported (supported: attention)")
            m = cls._sub(lr, "mixer")
            rot, mask = cls._sub(m, "rot"), cls._sub(m, "mask")
            heads, kv_heads = m.integer("heads"), m.integer("kv_heads")
            dim = m.integer("dim")
            att = GoridraAttention(heads, kv_heads, dim, m.integer("vdim"), m.number("scale", lo=0.0),
                                   rot.integer("dims", lo=2), rot.number("base", lo=0.0), mask.integer("size", hi=1 << 30),
                                   m.integer("kv_from", None, lo=0) if m.has("kv_from") else None)
            if heads % kv_heads:
                fail(EFORMAT, f"{m.origin}: {heads} heads are not a multiple of {kv_heads} key/value heads")
            if att.rot_dims % 2 or att.rot_dims > dim:
                fail(EFORMAT, f"{m.origin}: rot.dims {att.rot_dims} must be even and at most dim {dim}")
            if att.kv_from is not None:
                src = layers[att.kv_from].mixer if att.kv_from < i else None
                if src is None or src.kv_from is not None:
                    fail(EFORMAT, f"{m.origin}: kv_from {att.kv_from} must name an earlier layer with keys and values of its own")
                if (src.kv_heads, src.dim, src.vdim) != (kv_heads, dim, att.vdim):
                    fail(EFORMAT, f"{m.origin}: layer {att.kv_from}'s keys and values do not have this layer's head count and sizes")
            mlp = None
            if lr.has("mlp"):
                f = cls._sub(lr, "mlp")
                fk = f.string("kind")
                if fk == "dense":
                    mlp = GoridraMLP("dense", f.integer("ff"))
                elif fk == "moe":
                    router = cls._sub(f, "router")
                    groups = cls._sub(router, "groups")
                    mlp = GoridraMLP("moe", cls._sub(f, "expert").integer("ff"), router.integer("experts"), router.integer("top"),
                                     groups.integer("count"), groups.integer("keep"))
                    per = mlp.experts // mlp.groups
                    if mlp.experts % mlp.groups or mlp.keep > mlp.groups or mlp.top > mlp.keep * per:
                        fail(EFORMAT, f"{f.origin}: {mlp.experts} experts, {mlp.groups} groups of which {mlp.keep} are kept "
                                      f"and {mlp.top} choices do not fit together")
                else:
                    fail(ENOTSUP, f"{f.origin}: a feed-forward of kind '{fk}' is not supported (supported: dense, moe)")
            layers.append(GoridraLayer(kind, att, mlp))
        return cls(architecture=r.string("architecture"), vocab=r.integer("vocab", hi=1 << 24), width=r.integer("width"),
                   norm_eps=cls._sub(r, "norm").number("eps", lo=0.0), logit_softcap=r.number("logit_softcap", lo=0.0),
                   layers=tuple(layers), raw=obj)

    def to_dict(self):
        """The config.json content that reads back as this configuration."""
        return dict(self.raw)
