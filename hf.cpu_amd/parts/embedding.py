"""Token embedding and the output head."""
import torch

from .. import memory
from ..registry import register_part
from .base import ParamSpec, Part


@register_part("embedding", "lookup")
class Embedding(Part):
    """``x[t, :] = table[token[t], :]`` without scaling (src/model.c:566-571). ``scale``: the row is multiplied by it.
    ``sinusoid_base`` b: a position vector is added whose entry 2i is ``sin(p b^(-2i / width))`` and entry 2i + 1 the cosine
    of the same angle, p the token's position in its sequence (the angle is an fp32 product of the position and a frequency
    rounded from fp64)."""
    graph_safe = True


    def __init__(self, vocab_size, hidden_size, prefix="", weight="weight", scale=None, sinusoid_base=None):
        """The table is the tensor ``prefix + weight``."""
        super().__init__(prefix)
        self.V, self.E = vocab_size, hidden_size
        self.name = prefix + weight
        self.scale = None if scale is None else float(scale)
        self.sinusoid_base = None if sinusoid_base is None else float(sinusoid_base)
        self.table = self.inv_freq = None

    def param_specs(self):
        return [ParamSpec(self.name, (self.V, self.E))]

    def bind(self, params, ops):
        self.table = params[self.name]
        if self.sinusoid_base is not None:
            def table():
                i = torch.arange((self.E + 1) // 2, dtype=torch.float64)
                inv = torch.pow(torch.tensor(self.sinusoid_base, dtype=torch.float64), -2.0 * i / self.E)
                return memory.to_device(inv.to(torch.float32), ops.device, "frequencies of the position vector")
            self.inv_freq = ops.shared(("sinusoid frequencies", self.E, self.sinusoid_base), table)

    def forward(self, ops, step, out_x):
        with ops.section("embed"):
            if self.inv_freq is not None:
                ops.embed(self.table, step.tokens, out_x, scale=self.scale, positions=step.positions, inv_freq=self.inv_freq)
            else:
                ops.embed(self.table, step.tokens, out_x, scale=self.scale)


@register_part("head", "linear")
class LinearHead(Part):
    """``logits = W h`` in fp32, no bias (src/model.c:633-635). With ``tied`` the
    matrix is the embedding table unless the checkpoint holds one of its own, which
    then wins (src/model.c:156-158). ``softcap`` c > 0: ``logits <- c * tanh(logits / c)``. ``scale``: the logits are
    multiplied by it (before a soft cap). ``weight``: the matrix's name after ``prefix``."""
    graph_safe = True
    lazy_input_ok = True


    def __init__(self, vocab_size, hidden_size, tied, tied_to="", prefix="", softcap=None, scale=None, weight="weight"):
        super().__init__(prefix)
        self.V, self.E = vocab_size, hidden_size
        self.tied = bool(tied)
        self.tied_to = tied_to
        self.softcap = float(softcap) if softcap else 0.0
        self.scale = None if scale is None else float(scale)
        self.name = prefix + weight
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.name, (self.V, self.E), optional=self.tied)]

    def bind(self, params, ops):
        own = params.get(self.name)
        self.weight = own if own is not None else params[self.tied_to]

    def forward(self, ops, h, out_logits):
        with ops.section("head"):
            ops.gemm(h, self.weight, out_logits)
            if self.scale is not None and self.scale != 1.0:
                ops.scale_rows(out_logits, self.scale)
            if self.softcap > 0.0:
                ops.softcap(out_logits, self.softcap)
