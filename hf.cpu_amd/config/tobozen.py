"""The typed configuration of the Tobozen design.

config.json: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``, ``norm.groups`` and ``layers``, a list with one
object a layer: ``type`` (the kind of mixer), ``mixer`` (its sizes and constants) and ``mlp`` (null, or ``kind`` ``moe``
with ``expert.ff``, ``expert.limit``, ``router.experts``, ``router.top``). Mixers:

* ``mamba2``: ``heads``, ``vdim``, ``state``, ``groups``, ``conv`` (taps), ``norm_groups``
* ``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot.dims``, ``rot.base``, ``v_mix`` (true or absent)
* ``lightning``: ``heads``, ``dim``, ``vdim``, ``decay`` (one number a head)

Every size and constant of a model comes from there; layers may differ from one another in all of them, and come in
any order.
"""
from dataclasses import dataclass
from typing import Optional

from ..status import EFORMAT, ENOTSUP, fail
from .reader import KeyReader


@dataclass(frozen=True)
class TobozenMamba2:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class TobozenAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    v_mix: bool


@dataclass(frozen=True)
class TobozenLightning:
    heads: int
    dim: int
    vdim: int
    decay: tuple


@dataclass(frozen=True)
class TobozenMoE:
    ff: int
    limit: float
    experts: int
    top: int


@dataclass(frozen=True)
class TobozenLayer:
    type: str
    mixer: object
    mlp: Optional[TobozenMoE]


MIXERS = ("mamba2", "attention", "lightning")


@dataclass(frozen=True, eq=False)
class TobozenConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    norm_groups: int
    layers: tuple
    raw: dict                    # config.json as read (to_dict gives it back)

    @staticmethod
    def _sub(r, key):
        v = r.obj.get(key)
        if not isinstance(v, dict):
            fail(EFORMAT, f"{r.origin}: key '{key}' is missing or not an object")
        return KeyReader(v, f"{r.origin}: {key}")

    @classmethod
    def _mixer(cls, kind, m):
        if kind == "mamba2":
            mx = TobozenMamba2(m.integer("heads"), m.integer("vdim"), m.integer("state"), m.integer("groups"),
                               m.integer("conv", hi=8), m.integer("norm_groups"))
            if mx.heads % mx.groups:
                fail(EFORMAT, f"{m.origin}: {mx.heads} heads are not a multiple of {mx.groups} groups")
            if (mx.heads * mx.vdim) % mx.norm_groups:
                fail(EFORMAT, f"{m.origin}: {mx.heads * mx.vdim} inner values do not form {mx.norm_groups} equal runs")
            return mx
        if kind == "attention":
            rot = cls._sub(m, "rot")
            mx = TobozenAttention(m.integer("heads"), m.integer("kv_heads"), m.integer("dim"), m.integer("vdim"),
                                  m.number("scale", lo=0.0), rot.integer("dims", lo=2), rot.number("base", lo=0.0),
                                  m.boolean("v_mix", False))
            if mx.heads % mx.kv_heads:
                fail(EFORMAT, f"{m.origin}: {mx.heads} heads are not a multiple of {mx.kv_heads} key/value heads")
            if mx.rot_dims % 2 or mx.rot_dims > mx.dim:
                fail(EFORMAT, f"{m.origin}: rot.dims {mx.rot_dims} must be even and at most dim {mx.dim}")
            return mx
        heads = m.integer("heads")
        decay = m.obj.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or \
                any(isinstance(d, bool) or not isinstance(d, (int, float)) or not 0.0 <= d <= 1.0 for d in decay):
            fail(EFORMAT, f"{m.origin}: key 'decay' must list one number between 0 and 1 for each of the {heads} heads")
        return TobozenLightning(heads, m.integer("dim"), m.integer("vdim"), tuple(float(d) for d in decay))

    @classmethod
    def from_dict(cls, obj, origin="config.json"):
        r = KeyReader(obj, origin)
        raw_layers = obj.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            fail(EFORMAT, f"{origin}: key 'layers' is missing or not a list of layers")
        layers, mixed_width = [], None
        for i, lo in enumerate(raw_layers):
            lr = KeyReader(lo, f"{origin}: layers[{i}]")
            kind = lr.string("type")
            if kind not in MIXERS:
                fail(ENOTSUP, f"{lr.origin}: a mixer of type '{kind}' is not supported (supported: {', '.join(MIXERS)})")
            mixer = cls._mixer(kind, cls._sub(lr, "mixer"))
            if kind == "attention" and mixer.v_mix:
                if mixed_width is None:
                    mixed_width = mixer.kv_heads * mixer.vdim
                elif mixer.kv_heads * mixer.vdim != mixed_width:
                    fail(EFORMAT, f"{lr.origin}: values of {mixer.kv_heads * mixer.vdim} cannot be mixed with the first mixing "
                                  f"layer's {mixed_width}")
            mlp = None
            if lr.has("mlp"):
                f = cls._sub(lr, "mlp")
                fk = f.string("kind")
                if fk != "moe":
                    fail(ENOTSUP, f"{f.origin}: a feed-forward of kind '{fk}' is not supported (supported: moe)")
                expert, router = cls._sub(f, "expert"), cls._sub(f, "router")
                mlp = TobozenMoE(expert.integer("ff"), expert.number("limit", lo=0.0), router.integer("experts", hi=1024),
                                 router.integer("top", hi=64))
                if mlp.top > mlp.experts:
                    fail(EFORMAT, f"{f.origin}: {mlp.top} choices among {mlp.experts} experts")
            layers.append(TobozenLayer(kind, mixer, mlp))
        norm = cls._sub(r, "norm")
        cfg = cls(architecture=r.string("architecture"), vocab=r.integer("vocab", hi=1 << 24), width=r.integer("width"),
                  norm_eps=norm.number("eps", lo=0.0), norm_groups=norm.integer("groups"), layers=tuple(layers), raw=obj)
        if cfg.width % cfg.norm_groups:
            fail(EFORMAT, f"{origin}: width {cfg.width} does not form {cfg.norm_groups} equal runs (norm.groups)")
        return cfg

    def to_dict(self):
        """The config.json content that reads back as this configuration."""
        return dict(self.raw)
