"""Gitasun as a plan: the stream starts as the scaled embedding; every layer is pre-norm with RMS norms whose weight is one
number, and a branch's result is multiplied by one number for the whole model and by a vector of its own before it joins the
stream; the mixer is, layer by layer, attention through latents (``latent_attention``), a recurrence whose forget gate also
writes (``hgrn2``), or two mixers side by side whose weighted sum is the result (``parallel``: attention with biases, rescaled
rotary frequencies, soft-capped scores and sigmoid weights, beside gated linear attention); the feed-forward, where a layer
has one, is dense with the tanh gelu or a mixture of gated experts (softmax over the chosen logits) with a shared expert;
logits from a head of its own after the model's norm.

Tensor names: ``embed``, ``head``, ``final.norm``; ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.ls1``, ``l<i>.ls2``; ``l<i>.mix.*`` (``dq``, ``dq.norm``,
``uq``, ``dkv``, ``dkv.norm``, ``uk``, ``uv``, ``g``, ``o`` / ``q``, ``f``, ``f.b``, ``lower``, ``v``, ``norm``, ``o`` / ``left.{q,k,v}`` (+ ``.b``),
``left.{pb,g,o}``, ``right.{q,k,v,g,o,norm,a1,a2,a2.b}``); ``l<i>.mlp.{up,down}`` or ``l<i>.mlp.router`` (+ ``.b``),
``l<i>.mlp.e<n>.{gate,up,down}``, ``l<i>.mlp.shared.{gate,up,down}``.
"""
from ..config.gitasun import GitasunConfig
from ..plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..registry import register_architecture

EXPERT_ALPHA = 1.0            # an expert's gate half is g sigmoid(g), silu
EXPERT_NAMES = dict(gate="gate", up="up", down="down")


def _norm(cfg, name):
    return PartSpec("rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps, prefix=name, weight="", scalar=True))


def _rotary(rot, head_dim):
    scaling = None
    if rot.scaling is not None:
        scaling = dict(factor=rot.scaling.factor, low=rot.scaling.low, high=rot.scaling.high, original=rot.scaling.original)
    return PartSpec("rotary", dict(head_dim=head_dim, rot_dim=rot.dims, theta=rot.base, scaling=scaling))


def _mixer(cfg, lc, prefix):
    E, m = cfg.width, lc.mixer
    if lc.type == "latent_attention":
        # attention sees a head as [rotated part | latent]: the rotation acts on the first dimensions of such a head
        return PartSpec("latent_attention", dict(
            hidden_size=E, n_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, v_head_dim=m.vdim, kv_rank=m.kv_rank,
            q_rank=m.q_rank or None, scale=m.scale, eps=cfg.norm_eps, position=_rotary(m.rot, m.rot_dim + m.kv_rank), prefix=prefix))
    if lc.type == "hgrn2":
        return PartSpec("hgrn2", dict(hidden_size=E, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, eps=cfg.norm_eps, prefix=prefix))
    lt, rt = m.left, m.right
    left = PartSpec("attention", dict(
        hidden_size=E, n_heads=lt.heads, n_kv_heads=lt.kv_heads, head_dim=lt.dim, v_head_dim=lt.vdim, qkv_bias=True, window=0,
        scale=lt.scale, position=_rotary(lt.rot, lt.dim), out_gate=True, softcap=lt.softcap or None, weights="sigmoid",
        prefix=prefix + "left.",
        names=dict(q="q", k="k", v="v", o="o", g="g", q_bias="q.b", k_bias="k.b", v_bias="v.b", head_bias="pb")))
    right = PartSpec("gla", dict(hidden_size=E, n_heads=rt.heads, head_dim=rt.dim, v_head_dim=rt.vdim, tau=rt.tau, eps=cfg.norm_eps,
                                 decay_rank=rt.decay_rank or None, prefix=prefix + "right."))
    return PartSpec("side_by_side", dict(hidden_size=E, left=left, right=right, normed=False, left_scale=m.left_scale,
                                         right_scale=m.right_scale, prefix=prefix))


def _feed_forward(cfg, f, prefix):
    E = cfg.width
    if f.kind == "dense":
        return PartSpec("mlp", dict(hidden_size=E, intermediate_size=f.ff, activation="gelu_tanh", prefix=prefix,
                                    names=dict(up="up", down="down")))
    shared = None
    if f.shared_ff:
        shared = PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=f.shared_ff, prefix=prefix + "shared.", names=EXPERT_NAMES))
    return PartSpec("moe", dict(
        hidden_size=E, expert_size=f.ff, n_experts=f.experts, top=f.top, scoring="softmax_chosen", renormalize=True, weight_on="output",
        gated=dict(alpha=EXPERT_ALPHA, limit=0.0, shift=0.0), router_bias=True, shared=shared, prefix=prefix,
        names=dict(router="router", router_bias="router.b", gate="e{e}.gate", up="e{e}.up", down="e{e}.down")))


def gitasun_plan(cfg):
    E = cfg.width
    layers, schedule = [], []
    for l, lc in enumerate(cfg.layers):
        prefix = f"l{l}."
        parts = dict(norm1=_norm(cfg, prefix + "norm1"), mixer=_mixer(cfg, lc, prefix + "mix."))
        scales = {"mixer": "ls1"}
        if lc.mlp is not None:
            parts.update(norm2=_norm(cfg, prefix + "norm2"), feed_forward=_feed_forward(cfg, lc.mlp, prefix + "mlp."))
            scales["feed_forward"] = "ls2"
        block = PartSpec("prenorm", dict(hidden_size=E, branch_scale=cfg.residual_mult, layer_scales=scales, prefix=prefix))
        layers.append(LayerPlan.of(prefix, block, **parts))
        schedule.append(ScheduleEntry(l))
    return ModelPlan(
        hidden_size=E, vocab_size=cfg.vocab,
        embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab, hidden_size=E, prefix="", weight="embed", scale=cfg.embedding_scale)),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab, hidden_size=E, tied=False, prefix="", weight="head")),
    ).check()


register_architecture("Gitasun", GitasunConfig, gitasun_plan)
