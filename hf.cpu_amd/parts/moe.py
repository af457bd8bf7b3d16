"""Mixture of experts: a router that picks a few small feed-forward layers for every token."""
import torch

from .. import memory
from ..registry import make_part, register_part
from ..status import EINVAL, ENOTSUP, fail
from .base import ParamSpec, Part


@register_part("feed_forward", "moe")
class MixtureOfExperts(Part):
    """``x += sum over the chosen experts e of weight_e * Wdown_e act(Wup_e h)``.

    Router: logits ``z = Wrouter h`` as fp32 sums, scores ``softmax(z)`` over all experts (``scoring="sigmoid"``: the
    logistic function of each). The experts form ``n_groups`` equal runs of neighbours; a run scores as its best
    expert, and only experts of the ``keep_groups`` best runs can be chosen. The ``top`` best of those are chosen;
    their weights are their scores over the sum of the chosen scores + 1e-20 (``renormalize=False``: the scores
    themselves), times ``weight_scale``. Experts have no gate and no biases; ``activation`` as in the plain mlp.

    The experts' matrices are held stacked, [experts, ff, width] and [experts, width, ff]: one launch walks all of
    them (``Ops.moe_experts``). ``names``: the tensors' names after ``prefix`` (keys router, up, down; up and down are
    patterns with ``{e}`` for the expert's number).

    ``gated`` = dict(alpha, limit, shift): the experts are gated units, ``Wdown (g sigmoid(alpha g) (u + shift))`` with
    ``g = min(Wgate h', limit)``, ``u = clamp(Wup h', -limit, limit)`` (``limit`` <= 0: unbounded), and ``h' = weight_e h``:
    the weight scales the expert's input, not its output (``weight_on="input"``). The gate matrices are named by
    ``names["gate"]``; gate and up of an expert are held as one matrix: in blocks of 32 gate rows and 32 up rows where the
    expert's size is a multiple of 32 (the up product then forms the activation in its last lines), else gate rows first.
    Gated experts with ``weight_on="output"`` are plain gated units whose results are weighted: ``sum_e weight_e Wdown_e (g
    sigmoid(alpha g) (u + shift))`` with ``g = Wgate h``, ``u = Wup h`` (alpha 1, shift 0: ``silu(g) u``).

    ``scoring="softmax_chosen"``: the ``top`` experts with the largest logits, weighted by the softmax over the chosen logits
    alone. ``router_bias``: the router's logits are ``Wrouter h + b`` (the tensor named by ``names["router_bias"]``, fp32).
    ``shared``: the PartSpec of a feed-forward that every token passes beside its experts; its result is added."""
    graph_safe = True

    def __init__(self, hidden_size, expert_size, n_experts, top, n_groups=1, keep_groups=1, activation="relu2",
                 scoring="softmax", renormalize=True, weight_scale=1.0, prefix="", names=None, gated=None,
                 weight_on="output", router_bias=False, shared=None):
        super().__init__(prefix)
        if weight_on not in ("output", "input") or (weight_on == "input" and gated is None):
            fail(ENOTSUP, "moe: experts without a gate weigh their output; gated experts their input or their output")
        self.gated = None if gated is None else (float(gated["alpha"]), float(gated.get("limit", 0.0)), float(gated.get("shift", 0.0)),
                                                 expert_size % 32 == 0)
        self.weight_on = weight_on
        if activation not in ("gelu_erf", "gelu_tanh", "relu2"):
            fail(ENOTSUP, f"moe: activation '{activation}' is not implemented")
        if scoring not in ("softmax", "sigmoid", "softmax_chosen"):
            fail(ENOTSUP, f"moe: scoring '{scoring}' is not implemented")
        if n_experts % n_groups or not 0 < keep_groups <= n_groups:
            fail(EINVAL, f"moe: {n_experts} experts do not form {n_groups} equal groups of which {keep_groups} are kept")
        if not 0 < top <= keep_groups * (n_experts // n_groups):
            fail(EINVAL, f"moe: {top} choices among the {keep_groups * (n_experts // n_groups)} experts of the kept groups")
        self.E, self.F, self.n_experts, self.top = hidden_size, expert_size, n_experts, top
        self.n_groups, self.keep_groups = n_groups, keep_groups
        self.activation, self.scoring = activation, scoring
        self.renormalize, self.weight_scale = bool(renormalize), float(weight_scale)
        self.names = {"router": "router.weight", "up": "experts.{e}.up_proj.weight", "down": "experts.{e}.down_proj.weight",
                      "gate": "experts.{e}.gate_proj.weight"}
        self.names["router_bias"] = "router.bias"
        self.names.update(names or {})
        self.router_bias = bool(router_bias)
        self.shared = None if shared is None else make_part("feed_forward", shared)
        self.w_router = self.b_router = self.w_up = self.w_down = None

    def sub_parts(self):
        return [] if self.shared is None else [self.shared]

    def _name(self, key, e=None):
        return self.prefix + (self.names[key] if e is None else self.names[key].format(e=e))

    def param_specs(self):
        specs = [ParamSpec(self._name("router"), (self.n_experts, self.E))]
        if self.router_bias:
            specs.append(ParamSpec(self._name("router_bias"), (self.n_experts,), "vector", ("normal", 0.1)))
        for e in range(self.n_experts):
            specs += [ParamSpec(self._name("up", e), (self.F, self.E)), ParamSpec(self._name("down", e), (self.E, self.F))]
            if self.gated is not None:
                specs.append(ParamSpec(self._name("gate", e), (self.F, self.E)))
        return specs

    def bind(self, params, ops):
        self.w_router = params[self._name("router")]
        self.b_router = params[self._name("router_bias")].contiguous() if self.router_bias else None
        ups = [params.pop(self._name("up", e)) for e in range(self.n_experts)]
        if self.gated is not None:                  # gate and up of an expert in one matrix: one product gives both
            gates = [params.pop(self._name("gate", e)) for e in range(self.n_experts)]
            if self.gated[3]:
                ups = [ops.interleave_experts(g.unsqueeze(0), u.unsqueeze(0))[0] for g, u in zip(gates, ups)]
            else:
                ups = [torch.cat([g, u], 0) for g, u in zip(gates, ups)]
            del gates
        downs = [params.pop(self._name("down", e)) for e in range(self.n_experts)]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in ups + downs) else ups[0].dtype
        self.w_up = memory.cat([m.to(dt).unsqueeze(0) for m in ups], 0, f"{self.prefix}up matrices of all experts")
        del ups
        self.w_down = memory.cat([m.to(dt).unsqueeze(0) for m in downs], 0, f"{self.prefix}down matrices of all experts")

    def forward(self, ops, step, h, x):
        T = h.shape[0]
        logits = ops.scratch("router_logits", (T, self.n_experts), torch.float32)
        with ops.section("router"):
            ops.gemm(h, self.w_router, logits, bias=self.b_router)
            ids, weights = ops.moe_route(logits, self.top, self.n_groups, self.keep_groups, self.scoring, self.renormalize,
                                         self.weight_scale)
        with ops.section("experts"):
            ops.moe_experts(h, ids, weights, self.w_up, self.w_down, self.activation, x, gated=self.gated, weight_on=self.weight_on)
        if self.shared is not None:
            with ops.section("shared_expert"):
                self.shared.forward(ops, step, h, x)
