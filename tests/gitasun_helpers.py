"""Shared by the Gitasun tests: small configurations that differ in every size and option, weights that give
activations of order one, model folders, and the plain implementation's logits."""
import json
import math
import os

import numpy as np

import helpers
import plain_gitasun as pg


def rot(dims, base=10000.0, scaling=None):
    r = dict(base=base, dims=dims)
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, scaling=None, scale=None, rot_dims=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, rot=rot(rot_dims or rot_dim, base, scaling),
             scale=scale if scale is not None else 1.3 / math.sqrt(dim + rot_dim))
    return dict(type="latent_attention", mixer=m)


def hgrn2(heads, dim, vdim):
    return dict(type="hgrn2", mixer=dict(heads=heads, dim=dim, vdim=vdim))


def left(heads, kv_heads, dim, vdim, rot_dims, base=10000.0, scaling=None, softcap=None, scale=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot=rot(rot_dims, base, scaling), scale=scale if scale is not None else 1.5 / math.sqrt(dim))
    if softcap is not None:
        m["softcap"] = softcap
    return m


def right(heads, dim, vdim, tau):
    return dict(heads=heads, dim=dim, vdim=vdim, tau=tau)


def parallel(lt, rt, left_scale=1.0, right_scale=1.0):
    return dict(type="parallel", mixer=dict(left=lt, right=rt, left_scale=left_scale, right_scale=right_scale))


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, shared=None):
    f = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    if shared is not None:
        f["shared"] = dict(ff=shared)
    return f


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def config(vocab, width, layers, eps=1e-6, embedding_scale=None, residual_mult=1.0):
    return dict(architecture="Gitasun", vocab=vocab, width=width, embedding=dict(scale=embedding_scale if embedding_scale is not None else math.sqrt(width)),
                residual_mult=residual_mult, norm=dict(eps=eps), layers=layers)


# Sizes that no matrix-core kernel takes (an odd width, heads of 5, 7, 10 and 12), a model that begins with a recurrence, a
# layer without a feed-forward, latents larger and smaller than the heads they expand to, a rotated part that is all of a head's
# rotation and one that is rotated only in part, one head and several, as many key/value heads as heads and fewer, rotation of
# a part of a head, frequencies rescaled and not, scores with a cap and without, one choice among the experts, several and all
# of them, with a shared expert and without, an expert size that is a multiple of 32 and others.
SMALL = config(131, 40, eps=1e-5, embedding_scale=3.0, residual_mult=0.8, layers=[
    layer(hgrn2(3, 5, 7), None),
    layer(latent(3, 6, 4, 5, 10, 7, base=100.0), moe(5, 3, 12)),
    layer(parallel(left(6, 3, 10, 6, 6, base=500.0, scaling=(4.0, 1.0, 3.0, 64), scale=0.3), right(2, 7, 9, 4.0), 0.7, 1.2), dense(24)),
    layer(latent(1, 8, 8, 12, 5, 9, base=50.0, scaling=(2.0, 1.0, 4.0, 32), rot_dims=6), dense(20)),
    layer(parallel(left(2, 2, 8, 8, 8, softcap=5.0), right(1, 12, 4, 1.0), -0.5, 1.0), moe(4, 1, 10, shared=6)),
    layer(hgrn2(1, 20, 4), moe(3, 3, 32, shared=8)),
])
# Sizes that the matrix-core kernels take: widths and heads that are multiples of 32, states of 64 x 64, 128 x 32, 32 x 64 and
# 64 x 128, experts of 64 and 96.
CORES = config(520, 256, residual_mult=0.6, layers=[
    layer(latent(4, 64, 32, 96, 96, 128), moe(8, 2, 64, shared=128)),
    layer(hgrn2(4, 64, 64), dense(512)),
    layer(parallel(left(8, 2, 64, 64, 32, base=40000.0, scaling=(6.0, 1.0, 3.0, 128), softcap=20.0), right(4, 32, 64, 8.0), 0.75, 1.25), moe(6, 3, 96)),
    layer(hgrn2(2, 128, 32), None),
    layer(latent(2, 32, 64, 128, 64, 64, base=1000.0), dense(256)),
    layer(parallel(left(4, 4, 32, 32, 32), right(2, 64, 128, 16.0), 1.0, 0.5), dense(320)),
])
CONFIGS = {"small": SMALL, "cores": CORES}
PAGE = {"small": 8, "cores": 16}
STORED = {"small": "F32", "cores": "BF16"}


def make_weights(cfg, seed):
    """name -> float32 array, every value a bfloat16 value (the engine in bf16 then holds what the plain implementation
    reads). Forget gates' biases and lower bounds are spread so that decays lie between a tenth and nearly one, the sigmoid
    attention's biases are negative (a key's weight is small unless its score is large), and the routers' biases are far
    enough apart that a rounding does not change a choice."""
    rng = np.random.default_rng(seed)
    E, V = cfg["width"], cfg["vocab"]

    def n(shape, std, mean=0.0):
        return helpers.bf16_round(mean + rng.standard_normal(shape) * std)

    def u(shape, lo, hi):
        return helpers.bf16_round(rng.uniform(lo, hi, shape))

    def gated(p, F):
        w[p + "gate"], w[p + "up"] = n((F, E), 1.3 / math.sqrt(E)), n((F, E), 1.3 / math.sqrt(E))
        w[p + "down"] = n((E, F), 1.0 / math.sqrt(F))

    w = {"embed": n((V, E), 0.7 / cfg["embedding"]["scale"]), "final.norm": n((), 0.1, 1.0), "head": n((V, E), 1.0 / math.sqrt(E))}
    for l, lc in enumerate(cfg["layers"]):
        p, m = f"l{l}.", lc["mixer"]
        for which in ("1",) + (("2",) if lc["mlp"] is not None else ()):
            w[p + "norm" + which] = n((), 0.15, 1.1)
            w[p + "ls" + which] = u(E, 0.3, 1.4)
        q = p + "mix."
        if lc["type"] == "latent_attention":
            H, D, R, P, C, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[q + "dq"], w[q + "dq.norm"] = n((Q, E), 1.0 / math.sqrt(E)), n(Q, 0.2, 1.0)
            w[q + "uq"] = n((H * (D + R), Q), 1.3 / math.sqrt(Q))
            w[q + "dkv"], w[q + "dkv.norm"] = n((C + R, E), 1.0 / math.sqrt(E)), n(C, 0.2, 1.0)
            w[q + "uk"], w[q + "uv"] = n((H * D, C), 1.3 / math.sqrt(C)), n((H * P, C), 1.0 / math.sqrt(C))
            w[q + "g"] = n((H * P, E), 1.2 / math.sqrt(E))
            w[q + "o"] = n((E, H * P), 1.0 / math.sqrt(H * P))
        elif lc["type"] == "hgrn2":
            H, D, P = m["heads"], m["dim"], m["vdim"]
            w[q + "q"], w[q + "f"], w[q + "v"] = n((H * D, E), 1.2 / math.sqrt(E)), n((H * D, E), 1.5 / math.sqrt(E)), n((H * P, E), 1.2 / math.sqrt(E))
            w[q + "f.b"], w[q + "lower"] = n(H * D, 1.5, 1.5), u(H * D, 0.0, 0.9)
            w[q + "norm"] = n(P, 0.2, 1.0)
            w[q + "o"] = n((E, H * P), 1.0 / math.sqrt(H * P))
        else:
            lt, rt = m["left"], m["right"]
            H, G, D, P = lt["heads"], lt["kv_heads"], lt["dim"], lt["vdim"]
            a = q + "left."
            for name, rows in (("q", H * D), ("k", G * D), ("v", G * P)):
                w[a + name], w[a + name + ".b"] = n((rows, E), 1.2 / math.sqrt(E)), n(rows, 0.3)
            w[a + "pb"] = n(H, 0.5, -3.0)
            w[a + "g"] = n((H * P, E), 1.2 / math.sqrt(E))
            w[a + "o"] = n((E, H * P), 1.0 / math.sqrt(H * P))
            H, D, P = rt["heads"], rt["dim"], rt["vdim"]
            a = q + "right."
            for name, rows in (("q", H * D), ("k", H * D), ("v", H * P), ("g", H * P)):
                w[a + name] = n((rows, E), 1.2 / math.sqrt(E))
            ra = 3 + l                                       # the decay's inner size: only the tensors tell
            w[a + "a1"], w[a + "a2"], w[a + "a2.b"] = n((ra, E), 1.0 / math.sqrt(E)), n((H * D, ra), 1.5 / math.sqrt(ra)), n(H * D, 1.5, 1.5)
            w[a + "norm"] = n(P, 0.2, 1.0)
            w[a + "o"] = n((E, H * P), 1.0 / math.sqrt(H * P))
        f = lc["mlp"]
        if f is None:
            continue
        q = p + "mlp."
        if f["kind"] == "dense":
            w[q + "up"], w[q + "down"] = n((f["ff"], E), 1.2 / math.sqrt(E)), n((E, f["ff"]), 1.0 / math.sqrt(f["ff"]))
        else:
            X = f["router"]["experts"]
            w[q + "router"] = n((X, E), 2.0 / math.sqrt(E))
            w[q + "router.b"] = helpers.bf16_round(rng.permutation(X) * 0.75)
            for e in range(X):
                gated(f"{q}e{e}.", f["expert"]["ff"])
            if f.get("shared") is not None:
                gated(q + "shared.", f["shared"]["ff"])
    return w


def make_model_dir(path, cfg, seed, weights=None, stored="F32"):
    """``stored``: F32 (a bf16 engine then keeps the matrices in 32-bit and runs the kernels for mixed operands) or
    BF16 (the kernels of the serving path)."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    helpers.write_safetensors(os.path.join(path, "model.safetensors"), weights if weights is not None else make_weights(cfg, seed), stored)
    return path


def random_requests(cfg, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab"], n)] for i, n in enumerate(lengths)}


def plain_logits(model_dir, reqs):
    cfg, w = pg.read_model(model_dir)
    return {r: pg.forward(cfg, w, toks) for r, toks in reqs.items()}


def random_config(rng, big):
    """A configuration drawn at random: two to six layers of every kind in any order, with sizes that the matrix-core
    kernels take (``big``) or that none of them takes."""
    def pick(*xs):
        return xs[int(rng.integers(0, len(xs)))]
    width = pick(128, 256, 384) if big else pick(24, 40, 56, 72, 100)
    layers = []
    for _ in range(int(rng.integers(2, 7))):
        kind = pick("latent", "hgrn2", "parallel")
        if kind == "latent":
            R = pick(32, 64) if big else pick(2, 4, 6, 10)
            mix = latent(pick(1, 2, 4), pick(32, 64, 128) if big else pick(3, 8, 11), R, pick(32, 64, 128) if big else pick(4, 9, 16),
                         pick(32, 64, 160) if big else pick(5, 12, 30), pick(32, 96) if big else pick(4, 13), base=pick(100.0, 10000.0),
                         scaling=pick(None, (4.0, 1.0, 4.0, 64)))
        elif kind == "hgrn2":
            mix = hgrn2(pick(1, 2, 4), pick(32, 64, 128) if big else pick(3, 8, 17, 24), pick(32, 64) if big else pick(4, 5, 12, 20))
        else:
            G = pick(1, 2, 4)
            D = pick(32, 64, 128) if big else pick(6, 10, 16, 24)
            lt = left(G * pick(1, 2, 3), G, D, D if big else pick(D, 4, 14), pick(D, D // 2 - (D // 2) % 2), base=pick(1000.0, 40000.0),
                      scaling=pick(None, (6.0, 1.0, 3.0, 128)), softcap=pick(None, 10.0, 25.0))
            rt = right(pick(1, 2, 4), pick(32, 64, 128) if big else pick(3, 8, 17, 24), pick(32, 64) if big else pick(4, 5, 12, 20), pick(1.0, 4.0, 12.0))
            mix = parallel(lt, rt, pick(1.0, 0.55, -0.4), pick(1.0, 1.15, 0.3))
        X = pick(2, 5, 8)
        ff = pick(None, dense(pick(32, 64, 96) if big else pick(4, 10, 24)),
                  moe(X, pick(1, 2, X), pick(32, 64, 96) if big else pick(4, 10, 32), shared=pick(None, 32 if big else 6)))
        layers.append(layer(mix, ff))
    return config(int(rng.integers(50, 400)), width, layers, eps=pick(1e-5, 1e-6), embedding_scale=pick(1.0, 4.0, math.sqrt(width)),
                  residual_mult=pick(1.0, 0.5, 0.8))
