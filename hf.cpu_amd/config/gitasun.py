"""The typed configuration of the Gitasun design.

config.json: ``architecture`` (the name), ``vocab``, ``width``, ``embedding.scale``, ``residual_mult``, ``norm.eps`` and ``layers``, a
list with one object a layer: ``type`` (the kind of mixer), ``mixer`` (its sizes and constants) and ``mlp`` (null, or a
feed-forward). Mixers:

* ``latent_attention``: ``heads``, ``dim`` (unrotated query/key dimensions a head), ``rot_dim`` (rotated ones), ``vdim``, ``kv_rank`` and
  ``q_rank`` (the latents' sizes; ``q_rank`` may be absent, the tensors then say), ``scale``, ``rot`` = {``base``, ``dims``, optionally
  ``scaling``}
* ``hgrn2``: ``heads``, ``dim``, ``vdim``
* ``parallel``: ``left`` (attention with sigmoid weights: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``softcap`` (absent or 0:
  none), ``rot`` = {``base``, ``dims``, optionally ``scaling`` = {``factor``, ``low``, ``high``, ``original``}}), ``right`` (gated linear
  attention: ``heads``, ``dim``, ``vdim``, ``tau``; optionally ``decay_rank``, the inner size of the decay's low-rank projection, which
  a checkpoint's tensors give otherwise), ``left_scale`` and ``right_scale``

Feed-forwards: ``kind`` ``dense`` with ``ff``, or ``moe`` with ``expert.ff``, ``router.experts``, ``router.top`` and optionally
``shared.ff`` (an expert that every token passes).

Every size and constant of a model comes from there; layers may differ from one another in all of them, and come in
any order.
"""
from dataclasses import dataclass
from typing import Optional

from ..status import EFORMAT, ENOTSUP, fail
from .reader import KeyReader


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class GitasunRotary:
    base: float
    dims: int
    scaling: Optional[RotaryScaling]


@dataclass(frozen=True)
class GitasunLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int          # 0: the tensors say
    scale: float
    rot: GitasunRotary


@dataclass(frozen=True)
class GitasunHgrn2:
    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class GitasunLeft:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float       # 0: none
    rot: GitasunRotary


@dataclass(frozen=True)
class GitasunRight:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int      # 0: the tensors say


@dataclass(frozen=True)
class GitasunParallel:
    left: GitasunLeft
    right: GitasunRight
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class GitasunMLP:
    kind: str            # dense | moe
    ff: int              # the dense layer's size, or an expert's
    experts: int = 0
    top: int = 0
    shared_ff: int = 0   # 0: no shared expert


@dataclass(frozen=True)
class GitasunLayer:
    type: str
    mixer: object
    mlp: Optional[GitasunMLP]


MIXERS = ("latent_attention", "hgrn2", "parallel")


@dataclass(frozen=True, eq=False)
class GitasunConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    residual_mult: float
    norm_eps: float
    layers: tuple
    raw: dict                    # config.json as read (to_dict gives it back)

    @staticmethod
    def _sub(r, key):
        v = r.obj.get(key)
        if not isinstance(v, dict):
            fail(EFORMAT, f"{r.origin}: key '{key}' is missing or not an object")
        return KeyReader(v, f"{r.origin}: {key}")

    @classmethod
    def _rotary(cls, m, limit):
        r = cls._sub(m, "rot")
        dims = r.integer("dims", lo=2, hi=limit)
        if dims % 2:
            fail(EFORMAT, f"{r.origin}: key 'dims' must be even, got {dims}")
        scaling = None
        if r.has("scaling"):
            s = cls._sub(r, "scaling")
            scaling = RotaryScaling(s.number("factor", lo=0.0), s.number("low", lo=0.0), s.number("high", lo=0.0), s.number("original", lo=0.0))
            if not scaling.high > scaling.low:
                fail(EFORMAT, f"{s.origin}: 'high' must exceed 'low'")
        return GitasunRotary(r.number("base", lo=0.0), dims, scaling)

    @classmethod
    def _mixer(cls, kind, m):
        if kind == "latent_attention":
            rot_dim = m.integer("rot_dim", hi=256)
            return GitasunLatent(m.integer("heads", hi=1024), m.integer("dim", hi=512), rot_dim, m.integer("vdim", hi=512),
                                 m.integer("kv_rank", hi=4096), m.integer("q_rank", 0, lo=0, hi=1 << 16), m.number("scale", lo=0.0),
                                 cls._rotary(m, rot_dim))
        if kind == "hgrn2":
            return GitasunHgrn2(m.integer("heads"), m.integer("dim", hi=256), m.integer("vdim"))
        lt, rt = cls._sub(m, "left"), cls._sub(m, "right")
        dim = lt.integer("dim", hi=256)
        left = GitasunLeft(lt.integer("heads", hi=1024), lt.integer("kv_heads"), dim, lt.integer("vdim", hi=256), lt.number("scale", lo=0.0),
                           lt.number("softcap", 0.0) or 0.0, cls._rotary(lt, dim))
        if left.heads % left.kv_heads:
            fail(EFORMAT, f"{lt.origin}: {left.heads} heads are not a multiple of {left.kv_heads} kv_heads")
        if left.softcap < 0.0:
            fail(EFORMAT, f"{lt.origin}: key 'softcap' has an implausible value {left.softcap}")
        right = GitasunRight(rt.integer("heads"), rt.integer("dim", hi=256), rt.integer("vdim"), rt.number("tau", lo=0.0),
                             rt.integer("decay_rank", 0, lo=0))
        return GitasunParallel(left, right, m.number("left_scale"), m.number("right_scale"))

    @classmethod
    def _mlp(cls, f):
        kind = f.string("kind")
        if kind == "dense":
            return GitasunMLP("dense", f.integer("ff"))
        if kind != "moe":
            fail(ENOTSUP, f"{f.origin}: a feed-forward of kind '{kind}' is not supported (supported: dense, moe)")
        router = cls._sub(f, "router")
        experts = router.integer("experts", hi=1024)
        top = router.integer("top", hi=64)
        if top > experts:
            fail(EFORMAT, f"{router.origin}: {top} choices among {experts} experts")
        shared = cls._sub(f, "shared").integer("ff") if f.has("shared") else 0
        return GitasunMLP("moe", cls._sub(f, "expert").integer("ff"), experts, top, shared)

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
            if kind not in MIXERS:
                fail(ENOTSUP, f"{lr.origin}: a mixer of type '{kind}' is not supported (supported: {', '.join(MIXERS)})")
            mixer = cls._mixer(kind, cls._sub(lr, "mixer"))
            mlp = cls._mlp(cls._sub(lr, "mlp")) if lr.has("mlp") else None
            layers.append(GitasunLayer(kind, mixer, mlp))
        norm, emb = cls._sub(r, "norm"), cls._sub(r, "embedding")
        return cls(architecture=r.string("architecture"), vocab=r.integer("vocab", hi=1 << 24), width=r.integer("width"),
                   embedding_scale=emb.number("scale"), residual_mult=r.number("residual_mult", 1.0), norm_eps=norm.number("eps", lo=0.0),
                   layers=tuple(layers), raw=obj)

    def to_dict(self):
        """The config.json content that reads back as this configuration."""
        return dict(self.raw)
