"""Mobupel as a plan: the stream starts as the scaled embedding plus a sinusoidal position vector; every layer norms before
and after each sublayer and multiplies the sublayer's result by a sigmoid gate of the sublayer's input; the mixer is,
layer by layer, a matrix memory with exponential gates (``mlstm``) or two mixers side by side (``parallel``: softmax
attention with a short convolution, per-head norms, heads mixed after the softmax and an output gate, beside the gated
delta rule), followed where the layer has one by a dense feed-forward whose activation is a sum of normed powers;
logits from a head of its own, scaled.

Tensor names: ``embed``, ``head``, ``final.norm``; ``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.rg1`` (+ ``.b``),
``l<i>.rg2`` (+ ``.b``); ``l<i>.mix.*`` (``q``, ``k``, ``v``, ``g``, ``o``, ``norm``, ``i``, ``i.b``, ``f``, ``f.b`` / ``left.{q,k,v,g,o,talk}``,
``left.{q,k}.norm``, ``left.{q,k,v}.conv``, ``left.out``, ``right.{q,k,v,b,a1,a2,dt_bias,A_log,g1,g2,norm,o}``, ``right.{q,k,v}.conv``,
``right.out``); ``l<i>.mlp.{up,down,act}``.
"""
from ..config.mobupel import MobupelConfig
from ..plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..registry import register_architecture

SINUSOID_BASE = 10000.0       # of the position vector that joins the embedding
SIDES_SCALE = 0.5             # the parallel mixer is half the sum of its sides


def _norm(cfg, name):
    return PartSpec("rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps, prefix=name, weight=""))


def mobupel_plan(cfg):
    E = cfg.width
    layers, schedule = [], []
    for l, lc in enumerate(cfg.layers):
        prefix, m = f"l{l}.", lc.mixer
        if lc.type == "mlstm":
            mixer = PartSpec("mlstm", dict(
                hidden_size=E, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, gate_cap=m.gate_cap, eps=cfg.norm_eps,
                prefix=prefix + "mix.", names=dict(q="q", k="k", v="v", g="g", o="o", norm="norm", i="i", i_bias="i.b", f="f", f_bias="f.b")))
        else:
            lt, rt = m.left, m.right
            left = PartSpec("attention", dict(
                hidden_size=E, n_heads=lt.heads, n_kv_heads=lt.kv_heads, head_dim=lt.dim, v_head_dim=lt.vdim, qkv_bias=False, window=0,
                scale=lt.scale, position=PartSpec("none", dict(head_dim=lt.dim)), conv_taps=lt.conv, head_norm=cfg.norm_eps, talk=True,
                out_gate=True, prefix=prefix + "mix.left.",
                names=dict(q="q", k="k", v="v", o="o", g="g", talk="talk", q_norm="q.norm", k_norm="k.norm", q_conv="q.conv",
                           k_conv="k.conv", v_conv="v.conv")))
            right = PartSpec("gated_delta", dict(
                hidden_size=E, n_heads=rt.heads, n_qk_heads=rt.kv_heads, head_dim=rt.dim, v_head_dim=rt.vdim, conv_taps=rt.conv,
                eps=cfg.norm_eps, decay_rank=rt.decay_rank or None, gate_rank=rt.gate_rank or None, prefix=prefix + "mix.right."))
            mixer = PartSpec("side_by_side", dict(hidden_size=E, left=left, right=right, eps=cfg.norm_eps, scale=SIDES_SCALE,
                                                  prefix=prefix + "mix.", names=dict(left_norm="left.out", right_norm="right.out")))
        parts = dict(norm1=_norm(cfg, prefix + "norm1"), mixer=mixer, norm1b=_norm(cfg, prefix + "norm1b"))
        gates = {"mixer": ("rg1", "rg1.b")}
        if lc.ff is not None:
            parts.update(norm2=_norm(cfg, prefix + "norm2"), norm2b=_norm(cfg, prefix + "norm2b"),
                         feed_forward=PartSpec("mlp", dict(hidden_size=E, intermediate_size=lc.ff, activation="polynorm", eps=cfg.norm_eps,
                                                           prefix=prefix + "mlp.", names=dict(up="up", down="down", act="act"))))
            gates["feed_forward"] = ("rg2", "rg2.b")
        layers.append(LayerPlan.of(prefix, PartSpec("sandwich", dict(hidden_size=E, gates=gates, prefix=prefix)), **parts))
        schedule.append(ScheduleEntry(l))
    return ModelPlan(
        hidden_size=E, vocab_size=cfg.vocab,
        embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab, hidden_size=E, prefix="", weight="embed", scale=cfg.embedding_scale,
                                          sinusoid_base=SINUSOID_BASE)),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=E, tied=False, prefix="", weight="head", scale=cfg.logit_scale)),
    ).check()


register_architecture("Mobupel", MobupelConfig, mobupel_plan)
