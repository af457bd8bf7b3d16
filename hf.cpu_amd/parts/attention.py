"""Softmax attention over a paged key/value cache, with grouped heads and an
optional window."""
import math

import torch

from .. import memory

from ..registry import make_part, register_part
from ..status import EINVAL, fail
from .base import FixedState, PagedKV, ParamSpec, Part


@register_part("mixer", "attention")
class Attention(Part):
    """``q = Wq h + bq`` etc. (src/model.c:581-585); position encoding on q and k;
    for query head ``h`` the key/value head is ``h / (heads / kv_heads)``; scores
    ``dot(q, k) * scale`` over the visible keys, softmax in fp32, weighted sum of
    values (src/model.c:499-528); ``x += Wo att`` (src/model.c:606-609).

    A key at ``pk`` is visible to a query at ``pq`` iff ``0 <= pq - pk`` and, when
    ``window > 0``, ``pq - pk < window``, and, when ``mask_chunk > 0``, ``pq // mask_chunk == pk // mask_chunk``
    (runs of ``mask_chunk`` positions counted from the start of the sequence, wherever a prompt was cut).

    ``own_kv=False``: the mixer has no key and value projections and no cache of its own; the plan's schedule lets
    its entry read an earlier entry's cache (``ScheduleEntry.cache_of``), with its own queries, scale and mask.

    ``names`` gives the tensors' names after ``prefix`` (keys q, k, v, o, and q_bias, k_bias, v_bias, o_bias).

    A position encoding that enters the scores instead of the queries and keys has an
    attribute ``score_slopes`` (fp32 on the device, one per query head): the score then is
    ``dot(q, k) * scale + score_slopes[h] * (pk - pq)``.

    ``qk_norm`` = eps: queries and keys are RMS-normed over the whole projection (all heads at once) with the weights
    ``q_norm`` and ``k_norm`` (names in ``names``), before the rotation. ``sink``: the softmax has one more term of score 0
    that has no value, ``p_j = exp(s_j) / (1 + sum exp(s_i))``. ``v_mix``: ``"first"``: this layer's values, as projected,
    are kept for the step; ``"blend"``: ``v <- (1 - l) v + l v_first`` with the scalar tensor ``v_mix`` (name in
    ``names``) and the kept values of the same token; the blended values are what is cached. A ``"first"`` layer holds the
    scalar too, unused.

    ``conv_taps`` K >= 1: q, k and v pass a causal convolution over the last K tokens per channel straight after the
    projection (tensors ``q_conv``, ``k_conv``, ``v_conv`` in ``names``, [channels, K], the last column the current token's, no
    bias, zeros before a sequence's start); the last K - 1 projected rows of a request are part of its state, so the mixer
    then needs ``{"kv": PagedKV, "conv": FixedState}`` (one tap is a factor per channel and needs no state). ``head_norm`` = eps: queries and keys are RMS-normed head by head over
    ``head_dim`` with weights of that size which all heads share (``q_norm``, ``k_norm``). ``talk``: the heads' softmax weights
    are mixed after the softmax, ``weight_h <- sum_g talk[h, g] weight_g`` (tensor ``talk`` [heads, heads]), and head h applies
    its mixed weights to the values of its own group. ``out_gate``: the concatenated heads are multiplied by
    ``sigmoid(Wg h)`` (tensor ``g``) before the output projection. Any of the first three takes the mixer through a path of its
    own (``_forward_shaped``), which knows no rotation, no ``own_kv=False`` and none of ``qk_norm``, ``sink``, ``v_mix``; an output
    gate alone goes with every other option (its rows ride in the q/k/v product).
    ``forward(..., accumulate=False)`` writes ``x = ...`` instead of adding.

    ``softcap`` c > 0: a score becomes ``c tanh(score / c)`` after the scale. ``weights="sigmoid"``: no softmax; a visible key
    weighs ``sigmoid(score + b_h)`` with one number a head (the tensor ``head_bias`` in ``names``, [heads]), and the weights are
    not normalised over the keys.
    """
    graph_safe = True
    lazy_input_ok = True
    can_overwrite = True


    def __init__(self, hidden_size, n_heads, n_kv_heads, head_dim, qkv_bias, window, position,
                 scale=None, out_bias=False, v_head_dim=None, prefix="", mask_chunk=0, own_kv=True, names=None,
                 qk_norm=None, sink=False, v_mix=None, conv_taps=0, head_norm=None, talk=False, out_gate=False,
                 softcap=None, weights="softmax"):
        """``v_head_dim``: the size of a value head where it is not ``head_dim`` (key rows of the cache are
        then ``n_kv_heads * head_dim`` wide, value rows ``n_kv_heads * v_head_dim``, and the output
        projection reads ``n_heads * v_head_dim`` columns; such a mixer runs the plain kernels)."""
        super().__init__(prefix)
        if n_heads % n_kv_heads:
            fail(EINVAL, f"attention: {n_heads} heads are not a multiple of {n_kv_heads} key/value heads")
        self.E, self.H, self.G, self.D = hidden_size, n_heads, n_kv_heads, head_dim
        self.Dv = head_dim if v_head_dim is None else int(v_head_dim)
        self.QD, self.KD = n_heads * head_dim, n_kv_heads * head_dim
        self.VD, self.OD = n_kv_heads * self.Dv, n_heads * self.Dv
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = int(window)
        self.mask_chunk = int(mask_chunk)
        self.own_kv = bool(own_kv)
        self.names = {n: f"{n}_proj.weight" for n in "qkvo"}
        self.names.update({f"{n}_bias": f"{n}_proj.bias" for n in "qkvo"})
        self.names.update(q_norm="q_norm.weight", k_norm="k_norm.weight", v_mix="v_mix", talk="talk", g="g_proj.weight",
                          q_conv="q_conv.weight", k_conv="k_conv.weight", v_conv="v_conv.weight", head_bias="head_bias")
        self.names.update(names or {})
        self.conv_taps = int(conv_taps)
        self.head_norm = None if head_norm is None else float(head_norm)
        self.talk, self.out_gate = bool(talk), bool(out_gate)
        self.shaped = self.conv_taps >= 1 or self.head_norm is not None or self.talk
        self.softcap = float(softcap or 0.0)
        if weights not in ("softmax", "sigmoid") or self.softcap < 0.0 or (weights == "sigmoid" and sink):
            fail(EINVAL, f"attention: weights '{weights}' (softmax, or sigmoid without a sink term) and a soft cap of {softcap}")
        self.weights = weights
        self.head_bias = None
        if self.out_gate and not own_kv:
            fail(EINVAL, "attention: an output gate goes with a mixer that has projections of its own")
        if self.shaped and (position.kind != "none" or not own_kv or qk_norm is not None or sink or v_mix or qkv_bias or window
                            or mask_chunk or self.softcap or weights != "softmax"):
            fail(EINVAL, "attention: a convolution, per-head norms, mixed heads and an output gate go without rotation, biases, "
                         "windows and the other options")
        if not 0 <= self.conv_taps <= 8:
            fail(EINVAL, f"attention: a convolution over {self.conv_taps} tokens (at most 8)")
        self.taps = self.talk_w = self.no_state = None
        self.qk_norm = None if qk_norm is None else float(qk_norm)
        self.sink = bool(sink)
        if v_mix not in (None, "first", "blend") or (v_mix and not own_kv):
            fail(EINVAL, f"attention: v_mix '{v_mix}' is neither first nor blend, or the layer has no values of its own")
        self.v_mix = v_mix
        self.q_norm_w = self.k_norm_w = self.v_blend = None
        if self.window < 0 or self.mask_chunk < 0:
            fail(EINVAL, "attention: a window and a masking chunk are counted in tokens, 0 for none")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # src/model.c:507
        self.position = make_part("position", position)
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    def sub_parts(self):
        return [self.position]

    def param_specs(self):
        p, nm = self.prefix, self.names
        widths = {"q": self.QD, "k": self.KD, "v": self.VD}
        specs = [ParamSpec(p + nm[n], (widths[n], self.E)) for n in self._projections()]
        specs.append(ParamSpec(p + nm["o"], (self.E, self.OD)))
        if self.qkv_bias:
            specs += [ParamSpec(p + nm[n + "_bias"], (widths[n],), "vector") for n in self._projections()]
        if self.out_bias:
            specs.append(ParamSpec(p + nm["o_bias"], (self.E,), "vector"))
        if self.qk_norm is not None:
            specs.append(ParamSpec(p + nm["q_norm"], (self.QD,), "vector", ("one_plus_normal", 0.1)))
            if self.own_kv:
                specs.append(ParamSpec(p + nm["k_norm"], (self.KD,), "vector", ("one_plus_normal", 0.1)))
        if self.v_mix:
            specs.append(ParamSpec(p + nm["v_mix"], (), "vector", ("normal", 0.3), optional=self.v_mix == "first"))
        if self.conv_taps >= 1:
            specs += [ParamSpec(p + nm[n + "_conv"], (widths[n], self.conv_taps), "vector", ("normal", 0.3)) for n in "qkv"]
        if self.head_norm is not None:
            specs += [ParamSpec(p + nm[n], (self.D,), "vector", ("one_plus_normal", 0.1)) for n in ("q_norm", "k_norm")]
        if self.talk:
            specs.append(ParamSpec(p + nm["talk"], (self.H, self.H), "vector", ("normal", 0.3)))
        if self.out_gate:
            specs.append(ParamSpec(p + nm["g"], (self.OD, self.E)))
        if self.weights == "sigmoid":
            specs.append(ParamSpec(p + nm["head_bias"], (self.H,), "vector", ("normal", 0.5)))
        return specs

    def _projections(self):
        return "qkv" if self.own_kv else "q"

    def cache_need(self):
        if not self.own_kv:
            fail(EINVAL, f"attention '{self.prefix}' has no keys and values of its own: its schedule entry must read "
                         "another entry's cache")
        kv = PagedKV(self.KD, self.VD, self.window, self.mask_chunk)
        if self.conv_taps > 1:
            return {"kv": kv, "conv": FixedState((self.conv_taps - 1) * (self.QD + self.KD + self.VD))}
        return kv

    def reads_cache(self, need):
        """``need`` of the mixer whose storage this one reads, widened by what this one sees of it."""
        return PagedKV(need.k_width, need.v_width, need.window, need.mask_chunk, need.readers + ((self.window, self.mask_chunk),))

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        # One matrix for the three projections that share an input: rows of q, then k, then v.
        mats = [params[p + nm[n]] for n in self._projections()]
        if self.out_gate:
            mats.append(params[p + nm["g"]])             # the gate reads the same input: one product for all four
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = memory.cat([m.to(dt) for m in mats], 0, f"{p}q, k and v in one matrix")
        if self.qkv_bias:
            biases = [params[p + nm[n + "_bias"]] for n in self._projections()]
            if self.out_gate:                            # the gate's rows have none
                biases.append(torch.zeros(self.OD, dtype=biases[0].dtype, device=biases[0].device))
            self.b_qkv = memory.cat(biases, 0, f"{p}q, k and v biases in one vector")
        if self.weights == "sigmoid":
            self.head_bias = params[p + nm["head_bias"]].contiguous()
        self.w_o = params[p + nm["o"]]
        self.short_request_rows = ops.prompt_rows     # where the attention kernels for decoded tokens and for prompt portions part
        if self.out_bias:
            self.b_o = params[p + nm["o_bias"]]
        if self.qk_norm is not None:
            self.q_norm_w = params[p + nm["q_norm"]]
            self.k_norm_w = params[p + nm["k_norm"]] if self.own_kv else None
        if self.v_mix == "blend":
            self.v_blend = params[p + nm["v_mix"]].reshape(1)
        if self.conv_taps >= 1:
            self.no_state = memory.zeros((1, 1), torch.float32, ops.device, f"{p}a convolution's state that is never read")
            self.taps = memory.cat([params[p + nm[n + "_conv"]] for n in "qkv"], 0, f"{p}taps of q, k and v in one matrix").contiguous()
        if self.head_norm is not None:
            self.q_norm_w, self.k_norm_w = params[p + nm["q_norm"]].contiguous(), params[p + nm["k_norm"]].contiguous()
        if self.talk:
            self.talk_w = params[p + nm["talk"]].contiguous()
        elif self.out_gate and self.shaped:              # the gate rides in the kernel that mixes heads: an identity mix
            self.talk_w = memory.to_device(torch.eye(self.H, dtype=torch.float32), ops.device, f"{p}identity mix of heads")

    def _forward_shaped(self, ops, step, h, cache, x, accumulate):
        """The path of a mixer with a convolution, per-head norms, mixed heads or an output gate (see the class)."""
        T = h.shape[0]
        C = self.QD + self.KD + self.VD
        kv = cache["kv"] if isinstance(cache, dict) else cache
        proj = ops.scratch("qkv", (T, self.w_qkv.shape[0]), ops.act_dtype)
        with ops.section("qkv"):
            ops.gemm(h, self.w_qkv, proj)
        rows = proj[:, :C]
        with ops.section("qkv_prepare"):
            if self.conv_taps >= 1:
                rows = ops.scratch("qkv_conv", (T, C), torch.float32)
                ops.causal_conv(proj[:, :C], self.taps, None, cache["conv"].state if self.conv_taps > 1 else self.no_state, step, rows)
            q = ops.scratch("q_normed", (T, self.QD), ops.act_dtype)
            ops.head_norm_store(rows, self.H, self.G, self.D, self.Dv, self.q_norm_w, self.k_norm_w, self.head_norm or 0.0, q, kv,
                                step.group(kv.group).slot_map)
        att = ops.scratch("att", (T, self.OD), ops.act_dtype)
        with ops.section("attn"):
            if self.talk_w is None:
                ops.paged_attention(q, self.H, self.G, self.D, kv, step, 0, self.scale, att, v_head_dim=self.Dv)
            else:
                cross = ops.scratch("att_cross", (T, self.G * self.OD), ops.act_dtype)
                ops.paged_attention(q, self.H, self.G, self.D, kv, step, 0, self.scale, cross, v_head_dim=self.Dv, cross_values=True)
                ops.talk_mix(cross, self.talk_w, self.H, self.G, self.Dv, att, gate=proj[:, C:] if self.out_gate else None)
        with ops.section("wo"):
            if accumulate:
                ops.gemm(att, self.w_o, x, accumulate=True, defer=True)
            else:
                ops.gemm(att, self.w_o, x)

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        if self.shaped:
            if not write_cache:
                fail(EINVAL, f"attention '{self.prefix}': this mixer cannot read another entry's cache")
            return self._forward_shaped(ops, step, h, cache, x, accumulate)
        T = h.shape[0]
        if write_cache and not self.own_kv:
            fail(EINVAL, f"attention '{self.prefix}' has no keys and values to write")
        width = self.QD + self.KD + self.VD if write_cache else self.QD
        gate = None
        if self.out_gate:                       # [q | k | v | gate] from one product; a layer that only reads takes them apart
            if write_cache:
                rows = ops.scratch("qkv", (T, width + self.OD), ops.act_dtype)
                with ops.section("qkv"):
                    ops.gemm(h, self.w_qkv, rows, bias=self.b_qkv)
                qkv, gate = rows[:, :width], rows[:, width:]
            else:
                qkv = ops.scratch("qkv", (T, width), ops.act_dtype)
                gate = ops.scratch("att_gate", (T, self.OD), ops.act_dtype)
                with ops.section("qkv"):
                    ops.gemm(h, self.w_qkv[:width], qkv, bias=None if self.b_qkv is None else self.b_qkv[:width])
                    ops.gemm(h, self.w_qkv[self.w_qkv.shape[0] - self.OD:], gate)
        else:
            qkv = ops.scratch("qkv", (T, width), ops.act_dtype)
            # a product that split K is added up inside the next kernel (position.store, the next norm)
            with ops.section("qkv"):
                ops.gemm(h, self.w_qkv[:width], qkv, bias=None if self.b_qkv is None else self.b_qkv[:width], defer=True)
        prepare = {}
        if self.qk_norm is not None:
            prepare.update(q_norm=self.q_norm_w, k_norm=self.k_norm_w if write_cache else None, eps=self.qk_norm)
        if self.v_mix and write_cache:
            # the first mixing layer's values of this step's tokens wait in a work buffer for the layers that blend
            kept = ops.scratch("v_first", (T, self.VD), ops.act_dtype)
            prepare.update(dict(v_keep=kept) if self.v_mix == "first" else dict(v_blend=self.v_blend, v_other=kept))
        if prepare:
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache, v_head_dim=self.Dv,
                                prepare=prepare)
        elif self.Dv == self.D:
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache)
        else:                                   # only a position part that knows of value heads of another size can serve
            self.position.store(ops, step, qkv, self.H, self.G if write_cache else 0, cache, write_cache, v_head_dim=self.Dv)
        att = ops.scratch("att", (T, self.OD), ops.act_dtype)
        with ops.section("attn"):
            ops.paged_attention(qkv, self.H, self.G, self.D, cache, step, self.window, self.scale, att,
                                slopes=getattr(self.position, "score_slopes", None), v_head_dim=self.Dv,
                                mask_chunk=self.mask_chunk, sink=self.sink, softcap=self.softcap, weights=self.weights,
                                head_bias=self.head_bias)
            if gate is not None:
                ops.gate_mul(att, gate, att, "sigmoid")
        with ops.section("wo"):
            if accumulate:
                ops.gemm(att, self.w_o, x, bias=self.b_o, accumulate=True, defer=True)
            else:
                ops.gemm(att, self.w_o, x, bias=self.b_o)


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    """Causal softmax attention whose queries, keys and values come through latents. With H = ``n_heads``, D = ``head_dim`` (the
    unrotated dimensions of a query/key head), R = ``rot_dim`` (the rotated ones), Dv = ``v_head_dim``, C = ``kv_rank``:

    * ``c_q = rmsnorm(Wdq h) * q_norm``; ``q = Wuq c_q``, head by head ``[D unrotated | R rotated]``;
    * ``Wdkv h`` has ``C + R`` rows: the first C, RMS-normed with ``kv_norm``, are the latent ``c``; the last R are one key part
      that all heads share and that is rotated like the queries' R parts (``position``: a rotary PartSpec over R dimensions);
    * per head ``k = [Wuk c | rotated part]``, ``v = Wuv c``; ``score = q . k * scale``; softmax over the keys ``j <= i``;
    * the concatenated heads are multiplied by ``sigmoid(Wg h)`` (``out_gate``) and projected by ``Wo``.

    The cache holds one row a token: the rotated part and the latent as the key of one shared head, the latent as its value. The
    keys' expansion is folded into the queries, ``q' = Wuk_h^T q_h`` (``score = q' . c + q_rot . k_rot``), and the values' is
    applied after the weighted sum, ``o_h = Wuv_h (sum_j p_j c_j)``: attention itself is the engine's, with H query heads on one
    key/value head of ``R + C`` key and ``C`` value dimensions. The latents' norms are fp32 over the 32-bit sums of their products.
    ``names``: the tensors' names after ``prefix`` (keys dq, q_norm, uq, dkv, kv_norm, uk, uv, g, o).
    ``forward(..., accumulate=False)`` writes ``x = ...`` instead of adding."""
    graph_safe = True
    can_overwrite = True

    def __init__(self, hidden_size, n_heads, head_dim, rot_dim, v_head_dim, kv_rank, position, scale=None, q_rank=None, eps=1e-6,
                 out_gate=True, prefix="", names=None):
        """``q_rank`` None: the query latent's size is the tensors'."""
        super().__init__(prefix)
        self.E, self.H, self.D, self.R, self.Dv, self.C = hidden_size, n_heads, head_dim, rot_dim, v_head_dim, kv_rank
        self.q_rank = q_rank or None
        self.eps = float(eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim + rot_dim)
        self.out_gate = bool(out_gate)
        self.position = make_part("position", position)
        if getattr(self.position, "head_dim", rot_dim) != rot_dim + kv_rank:
            fail(EINVAL, f"latent_attention: the position part acts on heads of {rot_dim} + {kv_rank} dimensions, the rotated part first")
        self.names = dict(dq="dq", q_norm="dq.norm", uq="uq", dkv="dkv", kv_norm="dkv.norm", uk="uk", uv="uv", g="g", o="o")
        self.names.update(names or {})
        self.HD = rot_dim + kv_rank                          # a head as attention sees it: [rotated part | latent]
        self.w_down = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = self.q_norm_w = self.kv_norm_w = None

    def sub_parts(self):
        return [self.position]

    def param_specs(self):
        p, nm = self.prefix, self.names
        rq = self.q_rank or 0                                # 0: any size (the loader takes the tensor's)
        specs = [ParamSpec(p + nm["dq"], (rq, self.E)), ParamSpec(p + nm["q_norm"], (rq,), "vector", ("one_plus_normal", 0.1)),
                 ParamSpec(p + nm["uq"], (self.H * (self.D + self.R), rq), "matrix", ("normal", 0.1)),
                 ParamSpec(p + nm["dkv"], (self.C + self.R, self.E)),
                 ParamSpec(p + nm["kv_norm"], (self.C,), "vector", ("one_plus_normal", 0.1)),
                 ParamSpec(p + nm["uk"], (self.H * self.D, self.C), "matrix", ("normal", 0.1)),
                 ParamSpec(p + nm["uv"], (self.H * self.Dv, self.C), "matrix", ("normal", 0.1)),
                 ParamSpec(p + nm["o"], (self.E, self.H * self.Dv))]
        if self.out_gate:
            specs.append(ParamSpec(p + nm["g"], (self.H * self.Dv, self.E)))
        return specs

    def cache_need(self):
        return PagedKV(self.HD, self.C)

    def bind(self, params, ops):
        p, nm = self.prefix, self.names
        mats = [params[p + nm["dq"]], params[p + nm["dkv"]]]
        self.q_rank = mats[0].shape[0]
        if self.out_gate:
            self.w_gate = params[p + nm["g"]]
        dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        # the two projections into latents share their input: one product, whose 32-bit sums the norms read
        self.w_down = memory.cat([m.to(dt) for m in mats], 0, f"{p}both projections into latents in one matrix")
        self.w_uq, self.w_uv, self.w_o = params[p + nm["uq"]], params[p + nm["uv"]], params[p + nm["o"]]
        if self.w_uq.shape[1] != self.q_rank or params[p + nm["q_norm"]].numel() != self.q_rank:
            fail(EINVAL, f"latent_attention '{p}': the query latent's sizes do not match")
        # q' = Wuk_h^T q_h: the product reads Wuk_h [D, C] as [C, D] rows
        uk = params[p + nm["uk"]]
        self.w_uk_t = memory.to_device(uk.reshape(self.H, self.D, self.C).transpose(1, 2), ops.device,
                                       f"{p}the keys' expansion, transposed head by head")
        self.q_norm_w, self.kv_norm_w = params[p + nm["q_norm"]].contiguous(), params[p + nm["kv_norm"]].contiguous()
        self.short_request_rows = ops.prompt_rows

    def forward(self, ops, step, h, cache, x, write_cache=True, accumulate=True):
        if not write_cache:
            fail(EINVAL, f"latent_attention '{self.prefix}': this mixer cannot read another entry's cache")
        T, H, D, R, C, Dv, HD = h.shape[0], self.H, self.D, self.R, self.C, self.Dv, self.HD
        rq = self.q_rank
        down = ops.scratch("latent_down", (T, rq + C + R), torch.float32)
        with ops.section("latent_down"):
            ops.gemm(h, self.w_down, down)
            if self.out_gate:
                gate = ops.scratch("att_gate", (T, H * Dv), ops.act_dtype)
                ops.gemm(h, self.w_gate, gate)
        cq = ops.scratch("latent_q", (T, rq), ops.act_dtype)
        q = ops.scratch("latent_q_up", (T, H * (D + R)), ops.act_dtype)
        with ops.section("latent_q"):
            ops.group_rmsnorm(down[:, :rq], self.q_norm_w, self.eps, 1, cq)
            ops.gemm(cq, self.w_uq, q)
        packed = ops.scratch("qkv", (T, H * HD + HD + C), ops.act_dtype)
        folded = ops.scratch("latent_q_folded", (T, H * C), ops.act_dtype)
        with ops.section("latent_pack"):
            # the keys' expansion, folded into each head's query: one grouped product over the heads
            ops.head_products(q.view(T * H, D + R), self.w_uk_t, folded.view(T * H, C), H)
            ops.latent_pack(down[:, rq:], q, self.kv_norm_w, self.eps, packed, H, D, R, C, folded=folded)
            self.position.store(ops, step, packed, H, 1, cache, True, v_head_dim=C)
        att = ops.scratch("latent_att", (T, H * C), ops.act_dtype)
        with ops.section("latent_attn"):
            ops.paged_attention(packed, H, 1, HD, cache, step, 0, self.scale, att, v_head_dim=C)
        heads = ops.scratch("att", (T, H * Dv), ops.act_dtype)
        with ops.section("latent_v"):
            # the values' expansion of each head's weighted sum of latents
            ops.head_products(att.view(T * H, C), self.w_uv.view(H, Dv, C), heads.view(T * H, Dv), H)
            if self.out_gate:
                ops.gate_mul(heads, gate, heads, "sigmoid")
        with ops.section("latent_wo"):
            if accumulate:
                ops.gemm(heads, self.w_o, x, accumulate=True, defer=True)
            else:
                ops.gemm(heads, self.w_o, x)
