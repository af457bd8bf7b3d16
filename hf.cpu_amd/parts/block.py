"""Arrangements of a layer's parts around the residual stream."""
import torch

from ..registry import register_part
from .base import ParamSpec, Part


@register_part("block", "prenorm")
class PreNormBlock(Part):
    """``x += mixer(norm1(x)); x += feed_forward(norm2(x))`` (src/model.c:580-623):
    norms in front of each part, nothing after, the residual stream in fp32.

    ``branch_scale`` m and ``layer_scales`` = {"mixer": name, "feed_forward": name} (tensors of the model's width, after
    ``prefix``): a branch's result is multiplied by m and, element by element, by its vector before it joins the stream,
    ``x += m * ls * branch(norm(x))``. The branch's result, the factors and the sum are fp32: the branch is computed into a
    buffer of its own and added by one kernel."""
    graph_safe = True


    def __init__(self, hidden_size, prefix="", branch_scale=None, layer_scales=None):
        super().__init__(prefix)
        self.E = hidden_size
        self.branch_scale = None if branch_scale is None else float(branch_scale)
        self.scale_names = dict(layer_scales or {})
        self.scales = {}

    def param_specs(self):
        return [ParamSpec(self.prefix + n, (self.E,), "vector", ("one_plus_normal", 0.1)) for n in self.scale_names.values()]

    def bind(self, params, ops):
        self.scales = {k: params[self.prefix + n].contiguous() for k, n in self.scale_names.items()}

    def _scaled_branch(self, ops, x, which, part, run):
        """``x += branch_scale * layer_scale[which] * branch``; ``run(y, overwrite)`` makes the part write (or add) its result into ``y``."""
        y = ops.scratch("branch", (x.shape[0], self.E), torch.float32)
        if getattr(part, "can_overwrite", False):
            run(y, True)
        else:                                  # a part that only knows how to add: into zeros
            ops.settle()
            y.zero_()
            run(y, False)
        with ops.section("branch_sum"):
            ops.scale_add(y, x, scale=1.0 if self.branch_scale is None else self.branch_scale, columns=self.scales.get(which))

    def _forward_scaled(self, ops, step, x, parts, caches, write_cache):
        h = ops.scratch("normed", (x.shape[0], self.E), ops.act_dtype)
        parts["norm1"].forward(ops, x, h)
        ops.settle(x)
        mixer, cache = parts["mixer"], caches.get("mixer")
        self._scaled_branch(ops, x, "mixer", mixer, lambda y, over: mixer.forward(ops, step, h, cache, y, write_cache, accumulate=False)
                            if over else mixer.forward(ops, step, h, cache, y, write_cache))
        ff = parts.get("feed_forward")
        if ff is None:
            return
        parts["norm2"].forward(ops, x, h)
        ops.settle(x)
        self._scaled_branch(ops, x, "feed_forward", ff, lambda y, over: ff.forward(ops, step, h, y, accumulate=False)
                            if over else ff.forward(ops, step, h, y))

    def forward(self, ops, step, x, parts, caches, write_cache=True):
        """``parts``: norm1, mixer, norm2, feed_forward; ``caches``: the mixer's, under its name."""
        if self.branch_scale is not None or self.scale_names:
            return self._forward_scaled(ops, step, x, parts, caches, write_cache)
        h = ops.scratch("normed", (x.shape[0], self.E), ops.act_dtype)
        norm_for(ops, parts["norm1"], parts["mixer"], x, h)      # also adds up a product the previous part deferred into x
        ops.settle(x)                          # (nothing left to do unless the norm could not)
        parts["mixer"].forward(ops, step, h, caches.get("mixer"), x, write_cache)
        if "feed_forward" not in parts:         # a layer may be its mixer alone
            return
        norm_for(ops, parts["norm2"], parts["feed_forward"], x, h)
        ops.settle(x)
        parts["feed_forward"].forward(ops, step, h, x)


@register_part("block", "parallel")
class ParallelBlock(Part):
    """``h = norm1(x); x += mixer(h) + feed_forward(h)``: one norm, both branches read its output, and both sums go
    into the fp32 stream. A layer without a feed-forward has the mixer alone."""
    graph_safe = True

    def __init__(self, hidden_size, prefix=""):
        super().__init__(prefix)
        self.E = hidden_size

    def forward(self, ops, step, x, parts, caches, write_cache=True):
        """``parts``: norm1, mixer and, if the layer has one, feed_forward; ``caches``: the mixer's, under its name."""
        h = ops.scratch("normed", (x.shape[0], self.E), ops.act_dtype)
        parts["norm1"].forward(ops, x, h)            # also adds up a product that the layer before deferred into x
        ops.settle(x)
        parts["mixer"].forward(ops, step, h, caches.get("mixer"), x, write_cache)
        ff = parts.get("feed_forward")
        if ff is not None:
            ff.forward(ops, step, h, x)


@register_part("block", "sandwich")
class SandwichBlock(Part):
    """Norms before and after each sublayer: ``h = norm1(x); x += norm1b(gate(h) * mixer(h))``, then the same with ``norm2``,
    ``feed_forward`` and ``norm2b`` where the layer has a feed-forward. ``gate(h) = sigmoid(W h + b)`` multiplies the
    sublayer's result element by element before the second norm; ``gates`` names the tensors of each sublayer's gate after
    ``prefix``, ``{"mixer": (W, b), "feed_forward": (W, b)}`` (a sublayer that is not named has no gate). The sublayer's
    result, the gate, the second norm and the sum into the stream are fp32. The norms after the sublayers are parts with an
    ``add_into`` method (``rmsnorm``)."""
    graph_safe = True

    def __init__(self, hidden_size, gates=None, prefix=""):
        super().__init__(prefix)
        self.E = hidden_size
        self.gate_names = {k: tuple(v) for k, v in (gates or {}).items()}
        self.gate_w = {}

    def param_specs(self):
        specs = []
        for w, b in self.gate_names.values():
            specs += [ParamSpec(self.prefix + w, (self.E, self.E)), ParamSpec(self.prefix + b, (self.E,), "vector")]
        return specs

    def bind(self, params, ops):
        self.gate_w = {k: (params[self.prefix + w], params[self.prefix + b]) for k, (w, b) in self.gate_names.items()}

    def _sublayer(self, ops, step, x, h, which, part, post, run):
        """``x += post(gate(h) * part(h))``; ``run(y, overwrite)`` makes the part write (or add) its result into ``y``."""
        T = x.shape[0]
        y = ops.scratch("branch", (T, self.E), torch.float32)
        if getattr(part, "can_overwrite", False):
            run(y, True)
        else:                                  # a part that only knows how to add: into zeros
            ops.settle()
            y.zero_()
            run(y, False)
        gate = bias = None
        if which in self.gate_w:
            w, bias = self.gate_w[which]
            gate = ops.scratch("branch_gate", (T, self.E), torch.float32)
            with ops.section("gate"):
                ops.gemm(h, w, gate)
        with ops.section("post_norm"):
            post.add_into(ops, y, x, gate=gate, gate_bias=bias)

    def forward(self, ops, step, x, parts, caches, write_cache=True):
        """``parts``: norm1, mixer, norm1b and, if the layer has a feed-forward, norm2, feed_forward, norm2b."""
        h = ops.scratch("normed", (x.shape[0], self.E), ops.act_dtype)
        parts["norm1"].forward(ops, x, h)
        ops.settle(x)
        mixer, cache = parts["mixer"], caches.get("mixer")

        def run_mixer(y, overwrite):
            if overwrite:
                mixer.forward(ops, step, h, cache, y, write_cache, accumulate=False)
            else:
                mixer.forward(ops, step, h, cache, y, write_cache)
        self._sublayer(ops, step, x, h, "mixer", mixer, parts["norm1b"], run_mixer)
        ff = parts.get("feed_forward")
        if ff is None:
            return
        parts["norm2"].forward(ops, x, h)
        ops.settle(x)

        def run_ff(y, overwrite):
            if overwrite:
                ff.forward(ops, step, h, y, accumulate=False)
            else:
                ff.forward(ops, step, h, y)
        self._sublayer(ops, step, x, h, "feed_forward", ff, parts["norm2b"], run_ff)


def norm_for(ops, norm, reader, x, out, rows=None):
    """``out = norm(x)`` for the part ``reader``: lazily if the norm can be and the reader reads ``out`` through
    ``ops.gemm`` alone."""
    if getattr(norm, "can_be_lazy", False) and getattr(reader, "lazy_input_ok", False):
        norm.forward(ops, x, out, rows, lazy=True)
    else:
        norm.forward(ops, x, out, rows)
