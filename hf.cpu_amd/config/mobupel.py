"""The typed configuration of the Mobupel design.

config.json: ``architecture`` (the name), ``vocab``, ``width``, ``embedding.scale``, ``logit_scale``, ``norm.eps`` and ``layers``, a
list with one object a layer: ``type`` (the kind of mixer), ``mixer`` (its sizes and constants) and ``mlp`` (null, or ``kind``
``dense`` with ``ff``). Mixers:

* ``mlstm``: ``heads``, ``dim``, ``vdim``, ``gate_cap``
* ``parallel``: ``left`` (softmax attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``conv`` taps) and ``right`` (the
  gated delta rule: ``heads``, ``kv_heads`` heads of queries and keys, ``dim``, ``vdim``, ``conv`` taps; optionally ``decay_rank``
  and ``gate_rank``, the inner sizes of its two low-rank projections, which a checkpoint's tensors give otherwise and which
  only a folder of random weights needs)

Every size and constant of a model comes from there; layers may differ from one another in all of them, and come in
any order.
"""
from dataclasses import dataclass
from typing import Optional

from ..status import EFORMAT, ENOTSUP, fail
from .reader import KeyReader


@dataclass(frozen=True)
class MobupelMLSTM:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class MobupelLeft:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int


@dataclass(frozen=True)
class MobupelRight:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int         # 0: the tensors say
    gate_rank: int


@dataclass(frozen=True)
class MobupelParallel:
    left: MobupelLeft
    right: MobupelRight


@dataclass(frozen=True)
class MobupelLayer:
    type: str
    mixer: object
    ff: Optional[int]        # the dense feed-forward's size, None for a layer without one


MIXERS = ("mlstm", "parallel")


@dataclass(frozen=True, eq=False)
class MobupelConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    logit_scale: float
    norm_eps: float
    layers: tuple
    raw: dict                    # config.json as read (to_dict gives it back)

    @staticmethod
    def _sub(r, key):
        v = r.obj.get(key)
        if not isinstance(v, dict):
            fail(EFORMAT, f"{r.origin}: key '{key}' is missing or not an object")
        return KeyReader(v, f"{r.origin}: {key}")

    @staticmethod
    def _grouped(m, heads, kv_heads):
        if heads % kv_heads:
            fail(EFORMAT, f"{m.origin}: {heads} heads are not a multiple of {kv_heads} kv_heads")

    @classmethod
    def _mixer(cls, kind, m):
        if kind == "mlstm":
            return MobupelMLSTM(m.integer("heads"), m.integer("dim", hi=256), m.integer("vdim"), m.number("gate_cap", lo=0.0))
        lt, rt = cls._sub(m, "left"), cls._sub(m, "right")
        left = MobupelLeft(lt.integer("heads", hi=128), lt.integer("kv_heads"), lt.integer("dim", hi=256), lt.integer("vdim", hi=256),
                           lt.number("scale", lo=0.0), lt.integer("conv", hi=8))
        cls._grouped(lt, left.heads, left.kv_heads)
        right = MobupelRight(rt.integer("heads"), rt.integer("kv_heads"), rt.integer("dim", hi=256), rt.integer("vdim"),
                             rt.integer("conv", hi=8), rt.integer("decay_rank", 0, lo=0), rt.integer("gate_rank", 0, lo=0))
        cls._grouped(rt, right.heads, right.kv_heads)
        return MobupelParallel(left, right)

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
            ff = None
            if lr.has("mlp") and lo.get("mlp") is not None:
                f = cls._sub(lr, "mlp")
                fk = f.string("kind")
                if fk != "dense":
                    fail(ENOTSUP, f"{f.origin}: a feed-forward of kind '{fk}' is not supported (supported: dense)")
                ff = f.integer("ff")
            layers.append(MobupelLayer(kind, mixer, ff))
        norm, emb = cls._sub(r, "norm"), cls._sub(r, "embedding")
        return cls(architecture=r.string("architecture"), vocab=r.integer("vocab", hi=1 << 24), width=r.integer("width"),
                   embedding_scale=emb.number("scale"), logit_scale=r.number("logit_scale"), norm_eps=norm.number("eps", lo=0.0),
                   layers=tuple(layers), raw=obj)

    def to_dict(self):
        """The config.json content that reads back as this configuration."""
        return dict(self.raw)
