"""``bench.py --design goridra | tobozen | mobupel | gitasun``: prefill and decode of a design at sizes that resemble a real model's layers
(random weights), beside the closest other design at equal width, heads and layer count (Goridra beside Qwen2 dense,
Tobozen beside Goridra, Mobupel and Gitasun beside Tobozen), with every part of a step priced against its roofline: flops / time against the matrix cores
for a prefill's parts, bytes / time against HBM for a decode step's. One JSON line a size."""
import json
import math
import sys
import time

HBM_PEAK = 8.0e12
MFMA_PEAK = 2.5e15
PROMPT, PAGE = 2048, 16

# width, heads, key/value heads, head size, dense ff, experts, choices, groups, kept groups, expert ff, layers, vocabulary
# (for Tobozen also: heads, head size, state and groups of the state-space layers; layers come in threes; for Gitasun also the rotated
# part, the key/value latent and the query latent of its attention through latents)
SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=8192, experts=32, top=4, groups=4, keep=2, expert_ff=1024,
               layers=8, vocab=32000, mask=1024, ssm_heads=64, ssm_dim=64, ssm_state=128, ssm_groups=8, triples=2,
               latent_rot=64, latent_rank=512, latent_q=1536),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=14336, experts=64, top=8, groups=8, keep=4, expert_ff=1024,
               layers=4, vocab=32000, mask=1024, ssm_heads=128, ssm_dim=64, ssm_state=128, ssm_groups=8, triples=1,
               latent_rot=64, latent_rank=512, latent_q=1536),
}


def tobozen_shape(z):
    """Layers in threes: a state-space layer (inner width twice the model's), softmax attention, linear attention; each
    with a mixture of experts."""
    H, G, D = z["heads"], z["kv_heads"], z["dim"]
    moe = dict(kind="moe", expert=dict(ff=z["expert_ff"], limit=7.0), router=dict(experts=z["experts"], top=z["top"]))
    three = [
        dict(type="mamba2", mixer=dict(heads=z["ssm_heads"], vdim=z["ssm_dim"], state=z["ssm_state"], groups=z["ssm_groups"], conv=4,
                                       norm_groups=z["ssm_groups"]), mlp=moe),
        dict(type="attention", mixer=dict(heads=H, kv_heads=G, dim=D, vdim=D, scale=1.0 / math.sqrt(D), rot=dict(dims=D, base=500000.0),
                                          v_mix=True), mlp=moe),
        dict(type="lightning", mixer=dict(heads=H, dim=D, vdim=D, decay=[1.0 - 2.0 ** -(3 + 8 * h // H) for h in range(H)]), mlp=moe)]
    return dict(architecture="Tobozen", vocab=z["vocab"], width=z["width"], norm=dict(eps=1e-6, groups=2), layers=three * z["triples"])


def tobozen_work(z, T, batch, ctx):
    """({part: flops of a prefill of T tokens}, {part: bytes of a decode step}), all layers together, bf16. The
    recurrences are priced by the products of their state updates and outputs (4 N P a head and token) in a prefill and
    by their fp32 states, read and written once a request, in a decode step."""
    W, H, G, D, V, n3 = z["width"], z["heads"], z["kv_heads"], z["dim"], z["vocab"], z["triples"]
    QD, KD = H * D, G * D
    SH, SP, SN, SG = z["ssm_heads"], z["ssm_dim"], z["ssm_state"], z["ssm_groups"]
    inner = SH * SP
    w_in = 2 * inner + 2 * SG * SN + SH
    E, top, F = z["experts"], z["top"], z["expert_ff"]
    L = 3 * n3
    params = {"qkv": n3 * W * (QD + 2 * KD), "wo": n3 * QD * W, "ssm_in": n3 * W * w_in, "ssm_wo": n3 * inner * W,
              "lin_qkv": n3 * W * 4 * QD, "lin_wo": n3 * QD * W, "router": L * E * W, "head": V * W}
    pre = {k: 2.0 * T * v for k, v in params.items() if k != "head"}
    pre["attn"] = n3 * 4.0 * D * H * T * (T + 1) / 2
    pre["ssm_scan"] = n3 * T * SH * 4.0 * SN * SP
    pre["lin_scan"] = n3 * T * H * 4.0 * D * D
    pre["experts"] = L * T * top * 6.0 * F * W
    dec = {k: 2.0 * v for k, v in params.items()}
    touched = E * (1.0 - (1.0 - top / E) ** batch)
    dec["experts"] = L * touched * 3 * F * W * 2.0
    dec["attn"] = batch * ctx * 2 * KD * n3 * 2.0
    dec["ssm_scan"] = batch * n3 * SH * SN * SP * 4 * 2.0
    dec["lin_scan"] = batch * n3 * H * D * D * 4 * 2.0
    return pre, dec


def mobupel_shape(z):
    """Layers in pairs: two mixers side by side (softmax attention with mixed heads; the gated delta rule) with a dense
    feed-forward, then a matrix memory with exponential gates and no feed-forward."""
    H, G, D, W = z["heads"], z["kv_heads"], z["dim"], z["width"]
    pair = [
        dict(type="parallel", mixer=dict(
            left=dict(heads=H, kv_heads=G, dim=D, vdim=D, scale=1.0 / math.sqrt(D), conv=4),
            right=dict(heads=H, kv_heads=H, dim=D, vdim=D, conv=4, decay_rank=W // 32, gate_rank=W // 32)), mlp=dict(kind="dense", ff=z["ff"])),
        dict(type="mlstm", mixer=dict(heads=H, dim=D, vdim=D, gate_cap=15.0), mlp=None)]
    return dict(architecture="Mobupel", vocab=z["vocab"], width=W, embedding=dict(scale=math.sqrt(W)), logit_scale=1.0, norm=dict(eps=1e-6),
                layers=(pair * (3 * z["triples"]))[:3 * z["triples"]])


def mobupel_work(z, T, batch, ctx):
    """({part: flops of a prefill of T tokens}, {part: bytes of a decode step}), all layers together, bf16. Attention with
    mixed heads is priced as its scores once and its weights applied to the values of every group (what the identity that
    the kernels use costs); the recurrences by the products of their state updates and outputs (4 N P a head and token; the
    delta rule's correction is another 2 N P) in a prefill and by their fp32 states, read and written once a request, in a
    decode step."""
    W, H, G, D, V, F = z["width"], z["heads"], z["kv_heads"], z["dim"], z["vocab"], z["ff"]
    L = 3 * z["triples"]
    n2, n1 = (L + 1) // 2, L // 2                      # layers with two mixers side by side and a feed-forward; layers with a matrix memory
    QD, KD, r = H * D, G * D, W // 32
    params = {"qkv": n2 * W * (QD + 2 * KD + QD), "wo": n2 * QD * W, "delta_in": n2 * W * (3 * QD + H + 2 * r),
              "delta_low_rank": n2 * r * 2 * QD, "delta_wo": n2 * QD * W, "mlstm_in": n1 * W * (4 * QD + 2 * H), "mlstm_wo": n1 * QD * W,
              "gate": (2 * n2 + n1) * W * W, "up": n2 * F * W, "down": n2 * F * W, "head": V * W}
    pre = {k: 2.0 * T * v for k, v in params.items() if k != "head"}
    pre["attn"] = n2 * (2.0 + 2.0 * G) * D * H * T * (T + 1) / 2
    pre["delta_scan"] = n2 * T * H * 6.0 * D * D
    pre["mlstm_scan"] = n1 * T * H * 4.0 * D * (D + 1)
    dec = {k: 2.0 * v for k, v in params.items()}
    dec["attn"] = batch * ctx * 2 * KD * n2 * 2.0
    dec["delta_scan"] = batch * n2 * H * D * D * 4 * 2.0
    dec["mlstm_scan"] = batch * n1 * H * D * (D + 1) * 4 * 2.0
    return pre, dec


def gitasun_shape(z):
    """Layers in threes: attention through latents, a forget-gate recurrence, and two mixers side by side (attention with
    sigmoid weights; gated linear attention); each with a mixture of gated experts and a shared expert."""
    H, G, D, W = z["heads"], z["kv_heads"], z["dim"], z["width"]
    moe = dict(kind="moe", expert=dict(ff=z["expert_ff"]), router=dict(experts=z["experts"], top=z["top"]), shared=dict(ff=z["expert_ff"]))
    R, C = z["latent_rot"], z["latent_rank"]
    three = [
        dict(type="latent_attention", mixer=dict(heads=H, dim=D, rot_dim=R, vdim=D, kv_rank=C, q_rank=z["latent_q"], scale=1.0 / math.sqrt(D + R),
                                                 rot=dict(dims=R, base=10000.0)), mlp=moe),
        dict(type="hgrn2", mixer=dict(heads=H, dim=D, vdim=D), mlp=moe),
        dict(type="parallel", mixer=dict(
            left=dict(heads=H, kv_heads=G, dim=D, vdim=D, scale=1.0 / math.sqrt(D), softcap=50.0,
                      rot=dict(dims=D, base=500000.0, scaling=dict(factor=4.0, low=1.0, high=2.0, original=8192))),
            right=dict(heads=H, dim=D, vdim=D, tau=8.0, decay_rank=16), left_scale=0.5, right_scale=1.0), mlp=moe)]
    return dict(architecture="Gitasun", vocab=z["vocab"], width=W, embedding=dict(scale=math.sqrt(W)), residual_mult=0.5, norm=dict(eps=1e-6),
                layers=three * z["triples"])


def gitasun_work(z, T, batch, ctx):
    """({part: flops of a prefill of T tokens}, {part: bytes of a decode step}), all layers together, bf16. Attention through
    latents is priced as the engine computes it, H query heads on one key/value head of R + C key and C value dimensions; the
    recurrences by the products of their state updates and outputs (4 N P a head and token) in a prefill and by their fp32
    states, read and written once a request, in a decode step."""
    W, H, G, D, V, n3 = z["width"], z["heads"], z["kv_heads"], z["dim"], z["vocab"], z["triples"]
    R, C, Q = z["latent_rot"], z["latent_rank"], z["latent_q"]
    QD, KD = H * D, G * D
    E, top, F = z["experts"], z["top"], z["expert_ff"]
    L = 3 * n3
    params = {"latent_down": n3 * W * (Q + C + R + QD), "latent_q": n3 * Q * H * (D + R), "latent_pack": n3 * H * D * C, "latent_v": n3 * H * D * C,
              "latent_wo": n3 * QD * W, "qkv": n3 * W * (2 * QD + 2 * KD), "wo": n3 * QD * W, "forget_in": n3 * W * 3 * QD, "forget_wo": n3 * QD * W,
              "gla_in": n3 * (W * (4 * QD + 16) + 16 * QD), "gla_wo": n3 * QD * W, "router": L * E * W, "gate_up": L * 2 * F * W, "down": L * F * W, "head": V * W}      # (gate_up, down: the shared expert)
    pre = {k: 2.0 * T * v for k, v in params.items() if k != "head"}
    pre["latent_attn"] = n3 * 2.0 * (R + 2 * C) * H * T * (T + 1) / 2
    pre["attn"] = n3 * 4.0 * D * H * T * (T + 1) / 2
    pre["forget_scan"] = n3 * T * H * 4.0 * D * D
    pre["gla_scan"] = n3 * T * H * 4.0 * D * D
    pre["experts"] = L * T * top * 6.0 * F * W
    dec = {k: 2.0 * v for k, v in params.items()}
    touched = E * (1.0 - (1.0 - top / E) ** batch)
    dec["experts"] = L * touched * 3 * F * W * 2.0
    dec["latent_attn"] = batch * ctx * n3 * 2.0 * (R + 2 * C)
    dec["attn"] = batch * ctx * n3 * 2.0 * 2 * KD
    dec["forget_scan"] = batch * n3 * H * D * D * 4 * 2.0
    dec["gla_scan"] = batch * n3 * H * D * D * 4 * 2.0
    return pre, dec


def goridra_shape(z):
    """Layers in pairs: one with keys and values of its own and a dense feed-forward, one that reads them and has
    a mixture of experts."""
    def mixer(kv_from):
        m = dict(heads=z["heads"], kv_heads=z["kv_heads"], dim=z["dim"], vdim=z["dim"], scale=1.0 / math.sqrt(z["dim"]),
                 rot=dict(dims=z["dim"], base=500000.0), mask=dict(size=z["mask"]))
        if kv_from is not None:
            m["kv_from"] = kv_from
        return m
    layers = []
    for l in range(z["layers"]):
        if l % 2 == 0:
            layers.append(dict(type="attention", mixer=mixer(None), mlp=dict(kind="dense", ff=z["ff"])))
        else:
            layers.append(dict(type="attention", mixer=mixer(l - 1), mlp=dict(
                kind="moe", expert=dict(ff=z["expert_ff"]),
                router=dict(experts=z["experts"], top=z["top"], groups=dict(count=z["groups"], keep=z["keep"])))))
    return dict(architecture="Goridra", vocab=z["vocab"], width=z["width"], logit_softcap=30.0, norm=dict(eps=1e-6), layers=layers)


def qwen2_shape(z):
    """Qwen2 dense with the same width, heads and layer count; its gated feed-forward has the dense layer's matrices'
    worth of weights (three matrices of 2/3 the rows)."""
    return dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=z["layers"], hidden_size=z["width"],
                num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"], head_dim=z["dim"],
                intermediate_size=z["ff"] * 2 // 3 // 128 * 128, vocab_size=z["vocab"], rope_theta=500000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=True, use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu")


def part_work(design, z, T, batch, ctx):
    """({part: flops of a prefill of T tokens}, {part: bytes of a decode step of `batch` requests at context `ctx`}),
    all layers together, bf16."""
    if design == "tobozen":
        return tobozen_work(z, T, batch, ctx)
    if design == "mobupel":
        return mobupel_work(z, T, batch, ctx)
    if design == "gitasun":
        return gitasun_work(z, T, batch, ctx)
    W, H, G, D, L, V = z["width"], z["heads"], z["kv_heads"], z["dim"], z["layers"], z["vocab"]
    QD, KD = H * D, G * D
    if design == "qwen2":
        F = z["ff"] * 2 // 3 // 128 * 128
        params = {"qkv": L * W * (QD + 2 * KD), "wo": L * QD * W, "gate_up": L * 2 * F * W, "down": L * F * W, "head": V * W}
        pre = {k: 2.0 * T * v for k, v in params.items() if k != "head"}
        pre["attn"] = L * 4.0 * D * H * T * (T + 1) / 2
        dec = {k: 2.0 * v for k, v in params.items()}
        dec["attn"] = batch * ctx * 2 * KD * L * 2.0
        return pre, dec
    own, moe = (L + 1) // 2, L // 2
    seen = min(ctx % z["mask"] + 1, ctx)                         # keys of the current masking chunk
    E, top, F = z["experts"], z["top"], z["expert_ff"]
    params = {"qkv": W * (own * (QD + 2 * KD) + moe * QD), "wo": L * QD * W, "up": own * z["ff"] * W, "down": own * z["ff"] * W,
              "router": moe * E * W, "head": V * W}
    pre = {k: 2.0 * T * v for k, v in params.items() if k != "head"}
    pre["experts"] = moe * T * top * 4.0 * F * W
    chunk = z["mask"]
    pre["attn"] = L * 4.0 * D * H * sum(min(t % chunk + 1, t + 1) for t in range(T))
    dec = {k: 2.0 * v for k, v in params.items()}
    touched = E * (1.0 - (1.0 - top / E) ** batch)                # experts that a step of `batch` tokens reads, evenly routed
    dec["experts"] = moe * touched * 2 * F * W * 2.0
    dec["attn"] = batch * seen * 2 * KD * L * 2.0                 # readers walk their source's keys again
    return pre, dec


def run(args):
    import numpy as np
    import torch
    import hf_cpu_amd
    import hf_cpu_amd.session as S
    rng = np.random.default_rng(0)
    context = args.context
    for size in (args.sizes.split(",") if args.sizes else list(SIZES)):
        z = SIZES[size]
        line = {"size": size, "dims": z, "context": context, "dtype": "bf16", "data": "synthetic"}
        shapes = {"goridra": goridra_shape, "qwen2": qwen2_shape, "tobozen": tobozen_shape, "mobupel": mobupel_shape, "gitasun": gitasun_shape}
        beside = {"goridra": "qwen2", "tobozen": "goridra", "mobupel": "tobozen", "gitasun": "tobozen"}[args.design]
        if args.design in ("tobozen", "mobupel", "gitasun"):    # the same number of layers in both designs
            z = dict(z, layers=3 * z["triples"])
        for design, shape in ((args.design, shapes[args.design](z)), (beside, shapes[beside](z))):
            cfg = hf_cpu_amd.config_from_dict(shape)
            batches = [int(b) for b in args.batches.split(",")]
            room = -(-(args.steps + 16) // 64) * 64          # the decoded tokens: six to warm up, the timed ones, four profiled
            s = S.Session(cfg, dtype="bfloat16", ctx_max=context + room, batch=PROMPT, page_size=PAGE, max_seqs=max(batches),
                          kv_tokens=max(batches) * (context + room), seed=0)
            eng, ops = s.engine, s.ops

            def prompt(n=PROMPT):
                return [int(t) for t in rng.integers(0, z["vocab"], n)]
            out = {}
            times = []
            for rep in range(4):
                p = prompt()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                ops.argmax(eng.step([("p", p, [PROMPT - 1])])).cpu()
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                eng.release("p")
            pre_s = sorted(times[1:])[1]
            out["prefill_tok_per_s"] = round(PROMPT / pre_s, 1)
            eng.profile_start()
            for _ in range(2):
                eng.step([("p", prompt(), [PROMPT - 1])])
                eng.release("p")
            book = eng.profile_stop()["prefill"]
            pre_w, _ = part_work(design, z, PROMPT, 1, context)
            out["prefill_parts"] = {k: {"us": round(book.get(k, 0.0) / 2 * 1e3, 1),
                                        "frac": round(f / (book[k] / 2 * 1e-3) / MFMA_PEAK, 4)} for k, f in pre_w.items() if book.get(k)}
            out["prefill_parts"]["other"] = {"us": round(sum(v for k, v in book.items() if k not in pre_w) / 2 * 1e3, 1)}
            for batch in batches:
                ids = [("d", i) for i in range(batch)]
                for r in ids:
                    for at in range(0, context, PROMPT):
                        n = min(PROMPT, context - at)
                        eng.step([(r, prompt(n), [])])
                toks = [int(t) for t in rng.integers(0, z["vocab"], batch)]

                def one():
                    ops.argmax(eng.step([(r, [t], [0]) for r, t in zip(ids, toks)]))
                for _ in range(6):
                    one()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    one()
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t0) / args.steps
                _, dec_w = part_work(design, z, PROMPT, batch, context + 6 + args.steps // 2)
                out[f"decode_b{batch}_tok_per_s"] = round(batch / dt, 1)
                out[f"decode_b{batch}_ms"] = round(dt * 1e3, 4)
                out[f"decode_b{batch}_hbm_frac"] = round(sum(dec_w.values()) / dt / HBM_PEAK, 4)
                eng.profile_start()
                for _ in range(4):
                    one()
                book = eng.profile_stop()["decode"]
                out[f"decode_b{batch}_parts"] = {k: {"us": round(book.get(k, 0.0) / 4 * 1e3, 1),
                                                     "frac": round(b / (book[k] / 4 * 1e-3) / HBM_PEAK, 4)}
                                                 for k, b in dec_w.items() if book.get(k)}
                out[f"decode_b{batch}_parts"]["other"] = {"us": round(sum(v for k, v in book.items() if k not in dec_w) / 4 * 1e3, 1)}
                for r in ids:
                    eng.release(r)
            line[design] = out
            print(f"[bench] {size} {design}: prefill {out['prefill_tok_per_s']} tok/s, decode "
                  + ", ".join(f"b{b} {out[f'decode_b{b}_tok_per_s']} tok/s" for b in batches), file=sys.stderr, flush=True)
            del s, eng, ops
            torch.cuda.empty_cache()
        print(json.dumps(line), flush=True)
    return 0
