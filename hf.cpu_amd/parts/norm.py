"""Norms of the residual stream: root mean square with a learned scale (whole, or in groups), and layer norm with scale
and shift."""
from .. import memory
from ..registry import register_part
from ..status import EINVAL, fail
from .base import ParamSpec, Part


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """``y_i = x_i * (1 / sqrt(mean(x^2) + eps)) * w_i`` with the mean of squares in
    fp32 (src/mathx.c:65-75; the reference sums in fp64)."""
    graph_safe = True
    can_be_lazy = True          # forward(..., lazy=True) may leave the division to the products that read the output


    def __init__(self, size, eps, prefix="", weight="weight", scalar=False):
        """The scale is the tensor ``prefix + weight``; ``scalar``: a single number for all coordinates (a tensor without
        dimensions), held as a vector of that number."""
        super().__init__(prefix)
        self.size = size
        self.eps = float(eps)
        self.name = prefix + weight
        self.scalar = bool(scalar)
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.name, () if self.scalar else (self.size,), "vector", ("one_plus_normal", 0.1))]

    def bind(self, params, ops):
        self.weight = params[self.name]
        if self.scalar:
            self.weight = memory.to_device(self.weight.reshape(1).expand(self.size).contiguous(), ops.device,
                                           f"{self.name}, once a coordinate")

    def forward(self, ops, x, out, rows=None, lazy=False):
        """``out[r] = norm(x[rows[r]])`` (``rows`` None: every row in order). ``lazy``: the caller promises that
        ``out`` is read through ``ops.gemm`` alone (a part that says ``lazy_input_ok``); see ``Ops.rmsnorm``."""
        ops.rmsnorm(x, self.weight, self.eps, out, rows, lazy=lazy)

    def add_into(self, ops, y, x, gate=None, gate_bias=None, scale=1.0, accumulate=True):
        """``x (+)= scale * norm(y * sigmoid(gate + gate_bias))`` in fp32: the norm of a branch's result ``y`` (fp32) on its
        way into the stream (``gate`` None: ``y`` as it is)."""
        ops.rmsnorm_add(y, self.weight, self.eps, x, gate=gate, gate_bias=gate_bias, scale=scale, accumulate=accumulate)


@register_part("norm", "layernorm")
class LayerNorm(Part):
    """``y = (x - mean) / sqrt(var + eps) * w + b`` over the row, ``var`` the mean of the squared deviations, in fp32.
    ``weight`` and ``bias`` are the suffixes of the two tensors' names after ``prefix`` (``bias`` None: no shift)."""
    graph_safe = True

    def __init__(self, size, eps, weight="weight", bias="bias", prefix=""):
        super().__init__(prefix)
        self.size = size
        self.eps = float(eps)
        self.weight_name = prefix + weight
        self.bias_name = None if bias is None else prefix + bias
        self.weight = self.bias = None

    def param_specs(self):
        specs = [ParamSpec(self.weight_name, (self.size,), "vector", ("one_plus_normal", 0.1))]
        if self.bias_name is not None:
            specs.append(ParamSpec(self.bias_name, (self.size,), "vector", ("normal", 0.1)))
        return specs

    def bind(self, params, ops):
        self.weight = params[self.weight_name]
        self.bias = None if self.bias_name is None else params[self.bias_name]

    def forward(self, ops, x, out, rows=None):
        ops.layernorm(x, self.weight, self.bias, self.eps, out, rows)


@register_part("norm", "group_rmsnorm")
class GroupRMSNorm(Part):
    """The vector is cut into ``groups`` equal consecutive runs; each is divided by ``sqrt(mean(run^2) + eps)`` of its
    own, and the whole is multiplied by the weight. Sums in fp32. ``weight`` is the suffix of the tensor's name after
    ``prefix``. One group is the plain RMS norm (as a kernel of its own: nothing is left to the products around it).
    ``optional``: the tensor may be absent (a norm that a layer's arrangement never runs)."""
    graph_safe = True

    def __init__(self, size, eps, groups=1, weight="weight", prefix="", optional=False):
        super().__init__(prefix)
        self.optional = bool(optional)
        if groups <= 0 or size % groups:
            fail(EINVAL, f"group_rmsnorm: {size} values do not form {groups} equal runs")
        self.size, self.eps, self.groups = size, float(eps), int(groups)
        self.weight_name = prefix + weight
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.weight_name, (self.size,), "vector", ("one_plus_normal", 0.1), optional=self.optional)]

    def bind(self, params, ops):
        self.weight = params.get(self.weight_name) if self.optional else params[self.weight_name]

    def forward(self, ops, x, out, rows=None):
        ops.group_rmsnorm(x, self.weight, self.eps, self.groups, out, rows)
