"""Dense feed-forward parts."""
import torch

from .. import memory

from ..registry import register_part
from ..status import ENOTSUP, fail
from .base import ParamSpec, Part


@register_part("feed_forward", "gated_mlp")
class GatedMLP(Part):
    """``x += Wdown (act(Wgate h) * (Wup h))`` with ``act(g) = g / (1 + exp(-g))``
    (src/model.c:612-623, src/mathx.c:34). Gate and up share their input and are held
    as one matrix, gate rows first. ``names``: the tensors' names after ``prefix`` (keys gate, up, down)."""
    graph_safe = True
    lazy_input_ok = True


    def __init__(self, hidden_size, intermediate_size, activation="silu", prefix="", names=None):
        super().__init__(prefix)
        if activation != "silu":
            fail(ENOTSUP, f"gated_mlp: activation '{activation}' is not implemented")
        self.E, self.F = hidden_size, intermediate_size
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        self.names.update(names or {})
        self.w_gate_up = self.w_down = None
        self.fused = False

    def param_specs(self):
        p, nm = self.prefix, self.names
        return [ParamSpec(p + nm["gate"], (self.F, self.E)),
                ParamSpec(p + nm["up"], (self.F, self.E)),
                ParamSpec(p + nm["down"], (self.E, self.F))]

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        g, u = params[p + nm["gate"]], params[p + nm["up"]]
        dt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        # On the matrix cores gate and up rows are interleaved in blocks of 32, so that the product's
        # last step can form silu(gate) * up without storing gate and up.
        self.fused = ops.can_fuse_swiglu(g, u)
        if self.fused:
            memory.note(f"{p}gate and up, interleaved")
            self.w_gate_up = ops.interleave_gate_up(g, u)
        else:
            self.w_gate_up = memory.cat([g.to(dt), u.to(dt)], 0, f"{p}gate and up in one matrix")
        self.w_down = params[p + nm["down"]]

    def forward(self, ops, step, h, x):
        T = h.shape[0]
        act = ops.scratch("ffn_act", (T, self.F), ops.act_dtype)
        if self.fused:
            with ops.section("gate_up"):           # the activation is the product's last step
                ops.gemm(h, self.w_gate_up, act, swiglu=True)
        else:
            gu = ops.scratch("gate_up", (T, 2 * self.F), ops.act_dtype)
            with ops.section("gate_up"):
                ops.gemm(h, self.w_gate_up, gu)
            with ops.section("silu"):
                ops.swiglu(gu, act)
        with ops.section("down"):
            ops.gemm(act, self.w_down, x, accumulate=True, defer=True)


@register_part("feed_forward", "mlp")
class PlainMLP(Part):
    """``x += Wdown act(Wup h)`` without a gate: ``activation`` is ``gelu_erf`` (0.5 z (1 + erf(z / sqrt 2))),
    ``gelu_tanh`` or ``relu2`` (the square of relu), computed in fp32 on the product's rounded result, or ``polynorm``:
    ``a N(z) + b N(z^2) + c N(z^3) + e`` with the powers taken element by element, ``N`` dividing a token's vector by its
    root mean square (``eps`` inside the root) and ``(a, b, c, e)`` the tensor ``act``; its sums are fp32 over the product's
    32-bit result. ``names``: the tensors' names after ``prefix`` (keys up, down, act). ``forward(..., accumulate=False)``
    writes ``x = ...`` instead of adding."""
    graph_safe = True
    can_overwrite = True

    def __init__(self, hidden_size, intermediate_size, activation="gelu_erf", prefix="", names=None, eps=None):
        super().__init__(prefix)
        if activation not in ("gelu_erf", "gelu_tanh", "relu2", "polynorm"):
            fail(ENOTSUP, f"mlp: activation '{activation}' is not implemented")
        if activation == "polynorm" and eps is None:
            fail(ENOTSUP, "mlp: the activation of normed powers needs the norm's eps")
        self.E, self.F, self.activation = hidden_size, intermediate_size, activation
        self.eps = None if eps is None else float(eps)
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight", "act": "act"}
        self.names.update(names or {})
        self.w_up = self.w_down = self.coef = None

    def param_specs(self):
        specs = [ParamSpec(self.prefix + self.names["up"], (self.F, self.E)),
                 ParamSpec(self.prefix + self.names["down"], (self.E, self.F))]
        if self.activation == "polynorm":
            specs.append(ParamSpec(self.prefix + self.names["act"], (4,), "vector", ("normal", 0.5)))
        return specs

    def bind(self, params, ops):
        self.w_up = params[self.prefix + self.names["up"]]
        self.w_down = params[self.prefix + self.names["down"]]
        if self.activation == "polynorm":
            self.coef = params[self.prefix + self.names["act"]].contiguous()

    def forward(self, ops, step, h, x, accumulate=True):
        T = h.shape[0]
        act = ops.scratch("ffn_act", (T, self.F), ops.act_dtype)
        if self.activation == "polynorm":
            z = ops.scratch("ffn_up", (T, self.F), torch.float32)
            with ops.section("up"):
                ops.gemm(h, self.w_up, z)
            with ops.section("ffn_act"):
                ops.polynorm(z, self.coef, self.eps, act)
        else:
            with ops.section("up"):
                ops.gemm(h, self.w_up, act, activation=self.activation)
        with ops.section("down"):
            if accumulate:
                ops.gemm(act, self.w_down, x, accumulate=True, defer=True)
            else:
                ops.gemm(act, self.w_down, x)
