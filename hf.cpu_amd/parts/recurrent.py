"""Mixers that keep per-request state of fixed size instead of a growing cache: a state-space layer, linear
attention with a fixed decay, a matrix memory with exponential gates, recurrences with a decay per key channel (a forget gate
that also writes; gated linear attention), and the gated delta rule. All walk a request's
tokens in order from the state the step before left. The first three share one kernel for the recurrence
(``Ops.linear_scan``): ``S <- a_t S + k_t (b_t v_t)^T``, ``y_t = S^T q_t + d v_t``; the delta rule, whose write depends on
what the state already holds along the key, has its own (``Ops.delta_scan``). ``side_by_side`` runs two mixers on one
input and joins their normed results."""
import torch

from .. import memory
from ..kernels.ops import Ops
from ..registry import make_part, register_part
from ..status import EINVAL, fail
from .base import FixedState, ParamSpec, Part


@register_part("mixer", "mamba2")
class Mamba2(Part):
    """A state-space layer with a scalar decay per head and step. With ``inner = n_heads * head_dim``, N = ``state_size``
    and G = ``n_groups``, one projection of the input gives ``[z: inner | x: inner | B: G N | C: G N | dt: n_heads]``.
    ``x | B | C`` pass a causal convolution per channel over ``conv_taps`` inputs (the last tap is the current token's;
    zeros before a sequence's start) with a bias, and silu. ``dt <- softplus(dt + dt_bias)``. Per head h, with B and C of
    group ``h // (n_heads / G)``: ``S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T`` (S: N x head_dim),
    ``y_t = S_t^T C_t + D_h x_t``. Then ``y silu(z)`` is RMS-normed in ``norm_groups`` equal runs (weight ``norm``) and
    projected: ``x += Wo (...)``.

    Decays, step sizes, the recurrence and the norm are fp32; the state (S of every head, and the convolution's last
    ``conv_taps - 1`` inputs) is fp32 in the request's state row. ``names``: the tensors' names after ``prefix`` (keys
    in, conv, conv_bias, dt_bias, a_log, d, norm, o)."""
    graph_safe = True

    def __init__(self, hidden_size, n_heads, head_dim, state_size, n_groups, conv_taps, norm_groups, eps, prefix="", names=None):
        super().__init__(prefix)
        if n_heads % n_groups:
            fail(EINVAL, f"mamba2: {n_heads} heads are not a multiple of {n_groups} groups")
        self.E, self.H, self.P, self.N, self.G, self.K = hidden_size, n_heads, head_dim, state_size, n_groups, conv_taps
        self.inner = n_heads * head_dim
        if norm_groups <= 0 or self.inner % norm_groups:
            fail(EINVAL, f"mamba2: {self.inner} inner values do not form {norm_groups} equal runs")
        self.norm_groups, self.eps = norm_groups, float(eps)
        self.C = self.inner + 2 * n_groups * state_size            # channels of the convolution
        self.W_in = 2 * self.inner + 2 * n_groups * state_size + n_heads
        self.n_scan = Ops.scan_state_floats(n_heads, state_size, head_dim)    # of the recurrence in a state row; the convolution's follow
        self.names = {"in": "in_proj.weight", "conv": "conv.weight", "conv_bias": "conv.bias", "dt_bias": "dt_bias",
                      "a_log": "A_log", "d": "D", "norm": "norm.weight", "o": "out_proj.weight"}
        self.names.update(names or {})
        self.w_in = self.taps = self.conv_bias = self.dt_bias = self.a_log = self.d = self.norm_w = self.w_o = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        return [ParamSpec(p + nm["in"], (self.W_in, self.E)),
                ParamSpec(p + nm["conv"], (self.C, self.K), "vector", ("normal", 0.3)),
                ParamSpec(p + nm["conv_bias"], (self.C,), "vector", ("normal", 0.1)),
                ParamSpec(p + nm["dt_bias"], (self.H,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["a_log"], (self.H,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["d"], (self.H,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["norm"], (self.inner,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["o"], (self.E, self.inner))]

    def cache_need(self):
        return FixedState(self.n_scan + (self.K - 1) * self.C)

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        self.w_in, self.w_o = params[p + nm["in"]], params[p + nm["o"]]
        self.taps, self.conv_bias = params[p + nm["conv"]].contiguous(), params[p + nm["conv_bias"]]
        self.dt_bias, self.a_log, self.d = params[p + nm["dt_bias"]], params[p + nm["a_log"]], params[p + nm["d"]]
        self.norm_w = params[p + nm["norm"]]

    def forward(self, ops, step, h, cache, x, write_cache=True):
        if not write_cache:
            fail(EINVAL, f"mamba2 '{self.prefix}': a state cannot be read without being advanced")
        T, inner, GN = h.shape[0], self.inner, self.G * self.N
        proj = ops.scratch("ssm_in", (T, self.W_in), ops.act_dtype)
        with ops.section("ssm_in"):
            ops.gemm(h, self.w_in, proj)
        xbc = ops.scratch("ssm_conv", (T, self.C), torch.float32)
        y = ops.scratch("ssm_y", (T, inner), torch.float32)
        with ops.section("ssm_conv"):
            ops.causal_conv(proj[:, inner:inner + self.C], self.taps, self.conv_bias, cache.state[:, self.n_scan:], step, xbc,
                            activation="silu")
        with ops.section("ssm_scan"):
            ops.linear_scan(xbc[:, inner + GN:], xbc[:, inner:inner + GN], xbc[:, :inner], self.G, self.N, self.H, self.P,
                            cache.state, step, y, step_size=proj[:, inner + self.C:], step_bias=self.dt_bias, a_log=self.a_log,
                            skip=self.d)
        gated = ops.scratch("ssm_gated", (T, inner), ops.act_dtype)
        with ops.section("ssm_norm"):
            ops.group_rmsnorm(y, self.norm_w, self.eps, self.norm_groups, gated, gate=proj[:, :inner], gate_kind="silu_before")
        with ops.section("ssm_wo"):
            ops.gemm(gated, self.w_o, x, accumulate=True, defer=True)


@register_part("mixer", "lightning")
class LightningAttention(Part):
    """Linear attention with a fixed decay per head: ``q = silu(Wq h)``, ``k = silu(Wk h)`` (``n_heads`` x ``head_dim``),
    ``v = silu(Wv h)`` (``n_heads`` x ``v_head_dim``); per head ``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``,
    no other scale. The heads together are RMS-normed (weight ``norm``), multiplied by ``sigmoid(Wg h)`` and projected:
    ``x += Wo (...)``. The state is fp32 in the request's state row, as are the recurrence and the norm. ``names``: the
    tensors' names after ``prefix`` (keys q, k, v, g, norm, o)."""
    graph_safe = True

    def __init__(self, hidden_size, n_heads, head_dim, v_head_dim, decay, eps, prefix="", names=None):
        super().__init__(prefix)
        decay = tuple(float(d) for d in decay)
        if len(decay) != n_heads or not all(0.0 <= d <= 1.0 for d in decay):
            fail(EINVAL, f"lightning: {n_heads} heads need as many decays between 0 and 1, got {len(decay)}")
        self.E, self.H, self.D, self.Dv = hidden_size, n_heads, head_dim, v_head_dim
        self.decay_values, self.eps = decay, float(eps)
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight",
                      "norm": "norm.weight", "o": "out_proj.weight"}
        self.names.update(names or {})
        self.w_qkv = self.w_g = self.w_o = self.norm_w = self.decay = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        QD, VD = self.H * self.D, self.H * self.Dv
        return [ParamSpec(p + nm["q"], (QD, self.E)), ParamSpec(p + nm["k"], (QD, self.E)), ParamSpec(p + nm["v"], (VD, self.E)),
                ParamSpec(p + nm["g"], (VD, self.E)), ParamSpec(p + nm["norm"], (VD,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["o"], (self.E, VD))]

    def cache_need(self):
        return FixedState(Ops.scan_state_floats(self.H, self.D, self.Dv))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm[n]] for n in "qkv"]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k and v in one matrix")
        self.w_g, self.w_o, self.norm_w = params[p + nm["g"]], params[p + nm["o"]], params[p + nm["norm"]]
        self.decay = memory.to_device(torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32), ops.device,
                                      f"{p}decays")

    def forward(self, ops, step, h, cache, x, write_cache=True):
        if not write_cache:
            fail(EINVAL, f"lightning '{self.prefix}': a state cannot be read without being advanced")
        T, QD, VD = h.shape[0], self.H * self.D, self.H * self.Dv
        qkv = ops.scratch("lin_qkv", (T, 2 * QD + VD), ops.act_dtype)
        gate = ops.scratch("lin_gate", (T, VD), ops.act_dtype)
        with ops.section("lin_qkv"):
            ops.gemm(h, self.w_qkv, qkv, activation="silu")
            ops.gemm(h, self.w_g, gate)
        o = ops.scratch("lin_o", (T, VD), torch.float32)
        with ops.section("lin_scan"):
            ops.linear_scan(qkv[:, :QD], qkv[:, QD:2 * QD], qkv[:, 2 * QD:], self.H, self.D, self.H, self.Dv, cache.state, step, o,
                            decay=self.decay)
        normed = ops.scratch("lin_normed", (T, VD), ops.act_dtype)
        with ops.section("lin_norm"):
            ops.group_rmsnorm(o, self.norm_w, self.eps, 1, normed, gate=gate, gate_kind="sigmoid_after")
        with ops.section("lin_wo"):
            ops.gemm(normed, self.w_o, x, accumulate=True, defer=True)


@register_part("mixer", "mlstm")
class MatrixLSTM(Part):
    """A matrix memory per head with exponential input gates and sigmoid forget gates, kept stable by a running maximum of
    the gates' logarithms: ``q = Wq h / sqrt(head_dim)``, ``k = Wk h`` (``n_heads`` x ``head_dim``), ``v = Wv h`` (``n_heads`` x
    ``v_head_dim``); per head ``li = cap tanh((Wi h + bi) / cap)``, ``lf = logsigmoid(cap tanh((Wf h + bf) / cap))``;
    ``m_t = max(lf + m_(t-1), li)`` with ``m_0 = 0``; ``S_t = exp(lf + m_(t-1) - m_t) S_(t-1) + exp(li - m_t) k v^T``, ``n_t`` alike
    with ``k`` alone; ``o_t = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)``. Each head's ``o`` is divided by its root mean square
    (``eps``), the heads together are multiplied by ``norm`` and by ``sigmoid(Wg h)``, and projected. The state (S, n and m of
    every head), the gates and the recurrence are fp32. ``names``: the tensors' names after ``prefix`` (keys q, k, v, g, o,
    norm, i, i_bias, f, f_bias). ``forward(..., accumulate=False)`` writes ``x = ...`` instead of adding."""
    graph_safe = True
    can_overwrite = True

    def __init__(self, hidden_size, n_heads, head_dim, v_head_dim, gate_cap, eps, prefix="", names=None):
        super().__init__(prefix)
        if not gate_cap > 0.0:
            fail(EINVAL, f"mlstm: the gates' cap {gate_cap} must be positive")
        self.E, self.H, self.D, self.Dv = hidden_size, n_heads, head_dim, v_head_dim
        self.cap, self.eps = float(gate_cap), float(eps)
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight", "o": "out_proj.weight",
                      "norm": "norm.weight", "i": "i_proj.weight", "i_bias": "i_proj.bias", "f": "f_proj.weight", "f_bias": "f_proj.bias"}
        self.names.update(names or {})
        self.w_in = self.w_gates = self.w_o = self.norm_w = self.i_bias = self.f_bias = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        QD, VD = self.H * self.D, self.H * self.Dv
        return [ParamSpec(p + nm["q"], (QD, self.E)), ParamSpec(p + nm["k"], (QD, self.E)), ParamSpec(p + nm["v"], (VD, self.E)),
                ParamSpec(p + nm["g"], (VD, self.E)), ParamSpec(p + nm["o"], (self.E, VD)),
                ParamSpec(p + nm["norm"], (VD,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["i"], (self.H, self.E)), ParamSpec(p + nm["i_bias"], (self.H,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["f"], (self.H, self.E)), ParamSpec(p + nm["f_bias"], (self.H,), "vector", ("normal", 0.5))]

    def cache_need(self):
        return FixedState(Ops.scan_state_floats(self.H, self.D, self.Dv, normalizer=True))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm[n]] for n in "qkvg"]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_in = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k, v and the output gate in one matrix")
        gates = [params[p + nm["i"]], params[p + nm["f"]]]
        self.w_gates = memory.cat([m.to(dt) for m in gates], 0, f"{p}both gates in one matrix")
        self.w_o, self.norm_w = params[p + nm["o"]], params[p + nm["norm"]]
        self.i_bias, self.f_bias = params[p + nm["i_bias"]].contiguous(), params[p + nm["f_bias"]].contiguous()

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        if not write_cache:
            fail(EINVAL, f"mlstm '{self.prefix}': a state cannot be read without being advanced")
        T, QD, VD, H = h.shape[0], self.H * self.D, self.H * self.Dv, self.H
        proj = ops.scratch("mlstm_in", (T, 2 * QD + 2 * VD), ops.act_dtype)
        gates = ops.scratch("mlstm_gates", (T, 2 * H), torch.float32)
        with ops.section("mlstm_in"):
            ops.gemm(h, self.w_in, proj)
            ops.gemm(h, self.w_gates, gates)
        o = ops.scratch("mlstm_o", (T, VD), torch.float32)
        denom = ops.scratch("mlstm_denom", (T, H), torch.float32)
        with ops.section("mlstm_scan"):
            ops.linear_scan(proj[:, :QD], proj[:, QD:2 * QD], proj[:, 2 * QD:2 * QD + VD], H, self.D, H, self.Dv, cache.state, step, o,
                            exp_gates=(gates[:, :H], gates[:, H:], self.i_bias, self.f_bias, self.cap), q_scale=self.D ** -0.5,
                            denom=denom)
        normed = ops.scratch("mlstm_normed", (T, VD), ops.act_dtype)
        with ops.section("mlstm_norm"):
            ops.group_rmsnorm(o, self.norm_w, self.eps, H, normed, gate=proj[:, 2 * QD + VD:], gate_kind="sigmoid_after",
                              row_scale=denom)
        with ops.section("mlstm_wo"):
            if accumulate:
                ops.gemm(normed, self.w_o, x, accumulate=True, defer=True)
            else:
                ops.gemm(normed, self.w_o, x)


@register_part("mixer", "gated_delta")
class GatedDelta(Part):
    """The gated delta rule: ``q = Wq h``, ``k = Wk h`` (``n_qk_heads`` x ``head_dim``), ``v = Wv h`` (``n_heads`` x ``v_head_dim``);
    each passes a causal convolution over ``conv_taps`` tokens per channel (no bias, zeros before a sequence's start) and
    silu; ``q`` and ``k`` are made unit vectors head by head (``x / sqrt(sum x^2 + 1e-6)``) and ``q`` is divided by
    ``sqrt(head_dim)``. Per head h (queries and keys of head ``h // (n_heads / n_qk_heads)``): a write strength
    ``beta = sigmoid(Wb h)``, a decay per key channel ``g = exp(-exp(A_log_h) softplus(Wa2 (Wa1 h) + dt_bias))``, and
    ``S <- g * S`` (row by row); ``u = beta (v - S^T k)``; ``S <- S + k u^T``; ``o = S^T q``: a token is read
    from the state that already holds it. Each head's ``o`` is RMS-normed over ``v_head_dim`` with a weight of that size which all heads share, multiplied
    by ``sigmoid(Wg2 (Wg1 h))`` and projected. The state (S of every head and the convolution's last ``conv_taps - 1`` inputs),
    decays, strengths, unit vectors and the recurrence are fp32. ``names``: the tensors' names after ``prefix`` (keys q, k, v,
    q_conv, k_conv, v_conv, b, a1, a2, dt_bias, a_log, g1, g2, norm, o). ``forward(..., accumulate=False)`` writes ``x = ...``."""
    graph_safe = True
    can_overwrite = True
    UNIT_EPS = 1e-6

    def __init__(self, hidden_size, n_heads, n_qk_heads, head_dim, v_head_dim, conv_taps, eps, decay_rank=None, gate_rank=None,
                 prefix="", names=None):
        """``decay_rank`` and ``gate_rank``: the inner sizes of the two low-rank projections (None: taken from the tensors)."""
        super().__init__(prefix)
        if n_heads % n_qk_heads:
            fail(EINVAL, f"gated_delta: {n_heads} heads are not a multiple of {n_qk_heads} heads of queries and keys")
        if not 1 <= conv_taps <= 8:
            fail(EINVAL, f"gated_delta: a convolution over {conv_taps} tokens (1 to 8)")
        self.E, self.H, self.G, self.N, self.P, self.K = hidden_size, n_heads, n_qk_heads, head_dim, v_head_dim, conv_taps
        self.eps = float(eps)
        self.ra, self.rg = decay_rank, gate_rank
        self.KD, self.VD = n_qk_heads * head_dim, n_heads * v_head_dim
        self.C = 2 * self.KD + self.VD
        self.n_scan = Ops.scan_state_floats(n_heads, head_dim, v_head_dim)
        self.names = {n: n for n in ("q", "k", "v", "b", "a1", "a2", "dt_bias", "g1", "g2", "norm", "o")}
        self.names.update(q_conv="q.conv", k_conv="k.conv", v_conv="v.conv", a_log="A_log")
        self.names.update(names or {})
        self.w_qkv = self.w_small = self.w_b = self.w_a2 = self.w_g2 = self.w_o = self.taps = self.dt_bias = self.a_log = self.norm_w = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        ra, rg = self.ra or 0, self.rg or 0              # 0: any size (the loader takes the tensor's)
        return [ParamSpec(p + nm["q"], (self.KD, self.E)), ParamSpec(p + nm["k"], (self.KD, self.E)), ParamSpec(p + nm["v"], (self.VD, self.E)),
                ParamSpec(p + nm["q_conv"], (self.KD, self.K), "vector", ("normal", 0.3)),
                ParamSpec(p + nm["k_conv"], (self.KD, self.K), "vector", ("normal", 0.3)),
                ParamSpec(p + nm["v_conv"], (self.VD, self.K), "vector", ("normal", 0.3)),
                ParamSpec(p + nm["b"], (self.H, self.E)),
                ParamSpec(p + nm["a1"], (ra, self.E)), ParamSpec(p + nm["a2"], (self.H * self.N, ra), "matrix", ("normal", 0.1)),
                ParamSpec(p + nm["dt_bias"], (self.H * self.N,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["a_log"], (self.H,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["g1"], (rg, self.E)), ParamSpec(p + nm["g2"], (self.VD, rg), "matrix", ("normal", 0.1)),
                ParamSpec(p + nm["norm"], (self.P,), "vector", ("one_plus_normal", 0.1)),
                ParamSpec(p + nm["o"], (self.E, self.VD))]

    def cache_need(self):
        return FixedState(self.n_scan + (self.K - 1) * self.C)

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm[n]] for n in "qkv"]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k and v in one matrix")
        small = [params[p + nm[n]] for n in ("a1", "g1")]
        self.w_small = memory.cat([m.to(dt) for m in small], 0, f"{p}the low-rank projections' first halves in one matrix")
        self.w_b = params[p + nm["b"]]
        self.ra, self.rg = small[0].shape[0], small[1].shape[0]
        self.w_a2, self.w_g2, self.w_o = params[p + nm["a2"]], params[p + nm["g2"]], params[p + nm["o"]]
        if self.w_a2.shape[1] != self.ra or self.w_g2.shape[1] != self.rg:
            fail(EINVAL, f"gated_delta '{p}': the low-rank projections' inner sizes do not match")
        self.taps = memory.cat([params[p + nm[n + "_conv"]] for n in "qkv"], 0, f"{p}taps of q, k and v in one matrix").contiguous()
        self.dt_bias, self.a_log = params[p + nm["dt_bias"]].contiguous(), params[p + nm["a_log"]].contiguous()
        self.norm_w = memory.cat([params[p + nm["norm"]]] * self.H, 0, f"{p}the heads' norm weight, once a head")

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        if not write_cache:
            fail(EINVAL, f"gated_delta '{self.prefix}': a state cannot be read without being advanced")
        T, KD, VD, H = h.shape[0], self.KD, self.VD, self.H
        proj = ops.scratch("delta_in", (T, self.C), ops.act_dtype)
        small = ops.scratch("delta_small", (T, self.ra + self.rg), ops.act_dtype)
        beta = ops.scratch("delta_beta", (T, H), torch.float32)
        with ops.section("delta_in"):
            ops.gemm(h, self.w_qkv, proj)
            ops.gemm(h, self.w_small, small)
            ops.gemm(h, self.w_b, beta)
        a = ops.scratch("delta_decay", (T, H * self.N), torch.float32)
        gate = ops.scratch("delta_gate", (T, VD), ops.act_dtype)
        with ops.section("delta_low_rank"):
            ops.gemm(small[:, :self.ra], self.w_a2, a)
            ops.gemm(small[:, self.ra:], self.w_g2, gate)
        conv = ops.scratch("delta_conv", (T, self.C), torch.float32)
        with ops.section("delta_conv"):
            ops.causal_conv(proj, self.taps, None, cache.state[:, self.n_scan:], step, conv, activation="silu")
        y = ops.scratch("delta_y", (T, VD), torch.float32)
        with ops.section("delta_scan"):
            ops.delta_scan(conv[:, :KD], conv[:, KD:2 * KD], conv[:, 2 * KD:], self.G, self.N, H, self.P, a, self.dt_bias, self.a_log,
                           beta, cache.state, step, y, q_scale=self.N ** -0.5, unit_eps=self.UNIT_EPS)
        normed = ops.scratch("delta_normed", (T, VD), ops.act_dtype)
        with ops.section("delta_norm"):
            ops.group_rmsnorm(y, self.norm_w, self.eps, H, normed, gate=gate, gate_kind="sigmoid_after")
        with ops.section("delta_wo"):
            if accumulate:
                ops.gemm(normed, self.w_o, x, accumulate=True, defer=True)
            else:
                ops.gemm(normed, self.w_o, x)


@register_part("mixer", "hgrn2")
class ForgetGateRecurrence(Part):
    """Linear attention in which the forget gate also decides what is written: ``q = silu(Wq h)`` (``n_heads`` x ``head_dim``),
    ``v = Wv h`` (``n_heads`` x ``v_head_dim``), a forget gate per head and channel ``f = l + (1 - l) sigmoid(Wf h + b)`` with the
    lower bound ``l`` (tensor ``lower``, one value a (head, channel)); per head ``S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T``,
    ``o_t = S_t^T q_t`` (no key, no other scale). Each head's ``o`` is RMS-normed over ``v_head_dim`` with a weight of that size
    which all heads share, and the heads are projected. The gate, its complement, the state and the recurrence are fp32; the
    state lives in the request's state row. ``names``: the tensors' names after ``prefix`` (keys q, v, f, f_bias, lower, norm, o).
    ``forward(..., accumulate=False)`` writes ``x = ...`` instead of adding."""
    graph_safe = True
    can_overwrite = True

    def __init__(self, hidden_size, n_heads, head_dim, v_head_dim, eps, prefix="", names=None):
        super().__init__(prefix)
        self.E, self.H, self.D, self.Dv, self.eps = hidden_size, n_heads, head_dim, v_head_dim, float(eps)
        self.names = dict(q="q", v="v", f="f", f_bias="f.b", lower="lower", norm="norm", o="o")
        self.names.update(names or {})
        self.w_in = self.w_o = self.f_bias = self.lower = self.norm_w = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        QD, VD = self.H * self.D, self.H * self.Dv
        return [ParamSpec(p + nm["q"], (QD, self.E)), ParamSpec(p + nm["f"], (QD, self.E)), ParamSpec(p + nm["v"], (VD, self.E)),
                ParamSpec(p + nm["f_bias"], (QD,), "vector", ("normal", 0.5)), ParamSpec(p + nm["lower"], (QD,), "vector", ("normal", 0.2)),
                ParamSpec(p + nm["norm"], (self.Dv,), "vector", ("one_plus_normal", 0.1)), ParamSpec(p + nm["o"], (self.E, VD))]

    def cache_need(self):
        return FixedState(Ops.scan_state_floats(self.H, self.D, self.Dv))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm[n]] for n in ("q", "f", "v")]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_in = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, the forget gate and v in one matrix")
        self.w_o = params[p + nm["o"]]
        self.f_bias, self.lower = params[p + nm["f_bias"]].contiguous(), params[p + nm["lower"]].contiguous()
        self.norm_w = memory.cat([params[p + nm["norm"]]] * self.H, 0, f"{p}the heads' norm weight, once a head")

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        if not write_cache:
            fail(EINVAL, f"hgrn2 '{self.prefix}': a state cannot be read without being advanced")
        T, QD, VD = h.shape[0], self.H * self.D, self.H * self.Dv
        proj = ops.scratch("forget_in", (T, 2 * QD + VD), ops.act_dtype)
        with ops.section("forget_in"):
            ops.gemm(h, self.w_in, proj)
        o = ops.scratch("forget_o", (T, VD), torch.float32)
        with ops.section("forget_scan"):
            ops.channel_scan(proj[:, :QD], None, proj[:, 2 * QD:], self.H, self.D, self.Dv, proj[:, QD:2 * QD], self.f_bias, cache.state,
                             step, o, lower=self.lower, q_act="silu")
        normed = ops.scratch("forget_normed", (T, VD), ops.act_dtype)
        with ops.section("forget_norm"):
            ops.group_rmsnorm(o, self.norm_w, self.eps, self.H, normed)
        with ops.section("forget_wo"):
            if accumulate:
                ops.gemm(normed, self.w_o, x, accumulate=True, defer=True)
            else:
                ops.gemm(normed, self.w_o, x)


@register_part("mixer", "gla")
class GatedLinearAttention(Part):
    """Linear attention with a decay per key channel: ``q = Wq h / sqrt(head_dim)``, ``k = Wk h`` (``n_heads`` x ``head_dim``),
    ``v = Wv h`` (``n_heads`` x ``v_head_dim``), ``alpha = sigmoid(z)^(1 / tau)`` with ``z = Wa2 (Wa1 h) + b`` (a low-rank projection,
    one value a (head, key channel)); per head ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``. Each head's ``o``
    is RMS-normed over ``v_head_dim`` with a weight of that size which all heads share; the heads are multiplied by
    ``silu(Wg h)`` and projected. The decay (from ``z``'s 32-bit sums on: bias, logarithm of the sigmoid, the power), the state and
    the recurrence are fp32. ``names``: the tensors' names after ``prefix`` (keys q, k, v, g, o, norm, a1, a2, a2_bias).
    ``forward(..., accumulate=False)`` writes ``x = ...`` instead of adding."""
    graph_safe = True
    can_overwrite = True

    def __init__(self, hidden_size, n_heads, head_dim, v_head_dim, tau, eps, decay_rank=None, prefix="", names=None):
        """``decay_rank``: the inner size of the decay's low-rank projection (None: taken from the tensors)."""
        super().__init__(prefix)
        if not tau > 0.0:
            fail(EINVAL, f"gla: tau {tau} must be positive")
        self.E, self.H, self.D, self.Dv = hidden_size, n_heads, head_dim, v_head_dim
        self.tau, self.eps, self.ra = float(tau), float(eps), decay_rank or None
        self.names = dict(q="q", k="k", v="v", g="g", o="o", norm="norm", a1="a1", a2="a2", a2_bias="a2.b")
        self.names.update(names or {})
        self.w_in = self.w_a2 = self.w_o = self.a_bias = self.norm_w = None

    def param_specs(self):
        p, nm = self.prefix, self.names
        QD, VD, ra = self.H * self.D, self.H * self.Dv, self.ra or 0
        return [ParamSpec(p + nm["q"], (QD, self.E)), ParamSpec(p + nm["k"], (QD, self.E)), ParamSpec(p + nm["v"], (VD, self.E)),
                ParamSpec(p + nm["g"], (VD, self.E)), ParamSpec(p + nm["a1"], (ra, self.E)),
                ParamSpec(p + nm["a2"], (QD, ra), "matrix", ("normal", 0.1)), ParamSpec(p + nm["a2_bias"], (QD,), "vector", ("normal", 0.5)),
                ParamSpec(p + nm["norm"], (self.Dv,), "vector", ("one_plus_normal", 0.1)), ParamSpec(p + nm["o"], (self.E, VD))]

    def cache_need(self):
        return FixedState(Ops.scan_state_floats(self.H, self.D, self.Dv))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm[n]] for n in ("q", "k", "v", "g", "a1")]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_in = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k, v, the gate and the decay's first half in one matrix")
        self.ra = mats[4].shape[0]
        self.w_a2, self.w_o = params[p + nm["a2"]], params[p + nm["o"]]
        if self.w_a2.shape[1] != self.ra:
            fail(EINVAL, f"gla '{p}': the decay's low-rank projection has inner sizes {self.ra} and {self.w_a2.shape[1]}")
        self.a_bias = params[p + nm["a2_bias"]].contiguous()
        self.norm_w = memory.cat([params[p + nm["norm"]]] * self.H, 0, f"{p}the heads' norm weight, once a head")

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        if not write_cache:
            fail(EINVAL, f"gla '{self.prefix}': a state cannot be read without being advanced")
        T, QD, VD = h.shape[0], self.H * self.D, self.H * self.Dv
        proj = ops.scratch("gla_in", (T, 2 * QD + 2 * VD + self.ra), ops.act_dtype)
        z = ops.scratch("gla_decay", (T, QD), torch.float32)
        with ops.section("gla_in"):
            ops.gemm(h, self.w_in, proj)
            ops.gemm(proj[:, 2 * QD + 2 * VD:], self.w_a2, z)
        o = ops.scratch("gla_o", (T, VD), torch.float32)
        with ops.section("gla_scan"):
            ops.channel_scan(proj[:, :QD], proj[:, QD:2 * QD], proj[:, 2 * QD:2 * QD + VD], self.H, self.D, self.Dv, z, self.a_bias,
                             cache.state, step, o, tau=self.tau, q_scale=self.D ** -0.5)
        normed = ops.scratch("gla_normed", (T, VD), ops.act_dtype)
        with ops.section("gla_norm"):
            ops.group_rmsnorm(o, self.norm_w, self.eps, self.H, normed, gate=proj[:, 2 * QD + VD:2 * QD + 2 * VD], gate_kind="silu_after")
        with ops.section("gla_wo"):
            if accumulate:
                ops.gemm(normed, self.w_o, x, accumulate=True, defer=True)
            else:
                ops.gemm(normed, self.w_o, x)


@register_part("mixer", "side_by_side")
class SideBySide(Part):
    """Two mixers that read the same input; the result is ``scale * (norm_l(left(h)) + norm_r(right(h)))``, each side RMS-normed
    over the model's width with a weight of its own (``names``: keys left_norm, right_norm, after ``prefix``) before the sum
    (``scale`` 0.5: half the sum). ``left`` and ``right`` are PartSpecs of mixers; their caches are this mixer's, by the names
    ``left`` and ``right``. The sides' results, the norms and the sum are fp32. ``normed=False``: no norms and no weights; the result
    is the weighted sum ``left_scale * left(h) + right_scale * right(h)``."""
    graph_safe = True
    can_overwrite = True

    def __init__(self, hidden_size, left, right, eps=1e-6, scale=0.5, prefix="", names=None, normed=True, left_scale=1.0, right_scale=1.0):
        super().__init__(prefix)
        self.E, self.eps, self.scale = hidden_size, float(eps), float(scale)
        self.normed = bool(normed)
        self.side_scale = {"left": float(left_scale), "right": float(right_scale)}
        self.left, self.right = make_part("mixer", left), make_part("mixer", right)
        self.names = {"left_norm": "left.out", "right_norm": "right.out"}
        self.names.update(names or {})
        self.w_left = self.w_right = None
        self.short_request_rows = 0

    def sub_parts(self):
        return [self.left, self.right]

    def param_specs(self):
        if not self.normed:
            return []
        return [ParamSpec(self.prefix + self.names[n], (self.E,), "vector", ("one_plus_normal", 0.1)) for n in ("left_norm", "right_norm")]

    def cache_need(self):
        return {"left": self.left.cache_need(), "right": self.right.cache_need()}

    def bind(self, params, ops):
        if self.normed:
            self.w_left, self.w_right = params[self.prefix + self.names["left_norm"]], params[self.prefix + self.names["right_norm"]]
        self.short_request_rows = max(getattr(self.left, "short_request_rows", 0), getattr(self.right, "short_request_rows", 0))

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        T = h.shape[0]
        for side, w, name in ((self.left, self.w_left, "left"), (self.right, self.w_right, "right")):
            y = ops.scratch("side_" + name, (T, self.E), torch.float32)
            if getattr(side, "can_overwrite", False):
                side.forward(ops, step, h, cache[name], y, write_cache, accumulate=False)
            else:
                ops.settle()
                y.zero_()
                side.forward(ops, step, h, cache[name], y, write_cache)
            with ops.section("side_norm"):
                if self.normed:
                    ops.rmsnorm_add(y, w, self.eps, x, scale=self.scale, accumulate=accumulate or name == "right")
                else:
                    ops.scale_add(y, x, scale=self.side_scale[name], accumulate=accumulate or name == "right")
