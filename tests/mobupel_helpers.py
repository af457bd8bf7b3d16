"""Shared by the Mobupel tests: small configurations that differ in every size and option, weights that give
activations of order one, model folders, and the plain implementation's logits."""
import json
import math
import os

import numpy as np

import helpers
import plain_mobupel as pm


def mlstm(heads, dim, vdim, cap):
    return dict(type="mlstm", mixer=dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap))


def parallel(left, right):
    return dict(type="parallel", mixer=dict(left=left, right=right))


def left(heads, kv_heads, dim, vdim, conv, scale=None):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, scale=scale if scale is not None else 1.5 / math.sqrt(dim))


def right(heads, kv_heads, dim, vdim, conv):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)


def layer(mixer, ff):
    return dict(mixer, mlp=None if ff is None else dict(kind="dense", ff=ff))


def config(vocab, width, layers, eps=1e-6, embedding_scale=None, logit_scale=1.0):
    return dict(architecture="Mobupel", vocab=vocab, width=width, embedding=dict(scale=embedding_scale if embedding_scale is not None else math.sqrt(width)),
                logit_scale=logit_scale, norm=dict(eps=eps), layers=layers)


# Sizes that no matrix-core kernel takes (an odd width, heads of 10, 7 and 12 with value heads of another size), a model
# that begins with a matrix memory, two of them in a row, one with a feed-forward and a side-by-side layer without, as many
# key/value heads as heads and one, one to four taps (one tap: a factor a channel and no state), one head, a cap of 1.
SMALL = config(131, 40, eps=1e-5, embedding_scale=3.0, logit_scale=0.25, layers=[
    layer(mlstm(3, 6, 10, 5.0), None),
    layer(parallel(left(6, 3, 10, 6, 3, scale=0.4), right(4, 2, 7, 5, 2)), 24),
    layer(mlstm(1, 12, 4, 1.0), 20),
    layer(mlstm(2, 5, 5, 30.0), None),
    layer(parallel(left(4, 4, 8, 12, 1), right(3, 3, 12, 4, 4)), None),
    layer(parallel(left(5, 1, 6, 6, 4, scale=1.0), right(6, 1, 4, 9, 1)), 33),
])
# Sizes that the matrix-core kernels take: attention heads of 64, 32 and 128 whose values have the keys' size, in groups of
# two, one and two heads; states of 64 x 64, 128 x 32, 32 x 64 and 64 x 128.
CORES = config(520, 256, layers=[
    layer(parallel(left(8, 4, 64, 64, 3), right(4, 2, 64, 64, 4)), 320),
    layer(mlstm(4, 64, 64, 15.0), None),
    layer(parallel(left(4, 4, 32, 32, 2), right(2, 2, 128, 32, 3)), 512),
    layer(mlstm(2, 128, 64, 10.0), 256),
    layer(parallel(left(4, 2, 128, 128, 3), right(8, 4, 32, 64, 2)), None),
    layer(mlstm(8, 32, 32, 20.0), None),
])
CONFIGS = {"small": SMALL, "cores": CORES}
PAGE = {"small": 8, "cores": 16}
STORED = {"small": "F32", "cores": "BF16"}


def make_weights(cfg, seed):
    """name -> float32 array, every value a bfloat16 value (the engine in bf16 then holds what the plain implementation
    reads). Gates' biases, caps and decays are spread so that forget gates lie between a half and nearly one, input gates
    on both sides of the running maximum, and decays between a tenth and nearly one."""
    rng = np.random.default_rng(seed)
    E, V = cfg["width"], cfg["vocab"]

    def n(shape, std, mean=0.0):
        return helpers.bf16_round(mean + rng.standard_normal(shape) * std)

    w = {"embed": n((V, E), 0.7 / cfg["embedding"]["scale"] * math.sqrt(E) / math.sqrt(E)), "final.norm": n(E, 0.1, 1.0),
         "head": n((V, E), 1.0 / math.sqrt(E))}
    for l, lc in enumerate(cfg["layers"]):
        p, m = f"l{l}.", lc["mixer"]
        for which in ("1",) + (("2",) if lc["mlp"] is not None else ()):
            w[p + "norm" + which] = n(E, 0.1, 1.0)
            w[p + "norm" + which + "b"] = n(E, 0.1, 1.0)
            w[p + "rg" + which] = n((E, E), 1.5 / math.sqrt(E))
            w[p + "rg" + which + ".b"] = n(E, 0.5)
        if lc["type"] == "mlstm":
            H, D, P = m["heads"], m["dim"], m["vdim"]
            for name, rows in (("q", H * D), ("k", H * D), ("v", H * P), ("g", H * P)):
                w[p + "mix." + name] = n((rows, E), 1.2 / math.sqrt(E))
            w[p + "mix.o"] = n((E, H * P), 0.7 / math.sqrt(H * P))
            w[p + "mix.norm"] = n(H * P, 0.1, 1.0)
            w[p + "mix.i"] = n((H, E), 1.5 / math.sqrt(E))
            w[p + "mix.i.b"] = n(H, 0.5)
            w[p + "mix.f"] = n((H, E), 1.5 / math.sqrt(E))
            w[p + "mix.f.b"] = n(H, 1.0, 2.0)
        else:
            lt, rt = m["left"], m["right"]
            H, G, D, P, K = lt["heads"], lt["kv_heads"], lt["dim"], lt["vdim"], lt["conv"]
            q = p + "mix.left."
            for name, rows in (("q", H * D), ("k", G * D), ("v", G * P)):
                w[q + name] = n((rows, E), 1.2 / math.sqrt(E))
                w[q + name + ".conv"] = n((rows, K), 0.5)
            w[q + "q.norm"], w[q + "k.norm"] = n(D, 0.2, 1.0), n(D, 0.2, 1.0)
            w[q + "talk"] = n((H, H), 0.4) + helpers.bf16_round(np.eye(H) * 0.5)
            w[q + "g"] = n((H * P, E), 1.2 / math.sqrt(E))
            w[q + "o"] = n((E, H * P), 0.7 / math.sqrt(H * P))
            w[q + "out"] = n(E, 0.1, 1.0)
            H, G, N, P, K = rt["heads"], rt["kv_heads"], rt["dim"], rt["vdim"], rt["conv"]
            q = p + "mix.right."
            for name, rows in (("q", G * N), ("k", G * N), ("v", H * P)):
                w[q + name] = n((rows, E), 1.5 / math.sqrt(E))
                w[q + name + ".conv"] = n((rows, K), 0.6)
            ra, rg = 3 + l, 2 + 2 * l                       # the inner sizes of the low-rank projections: only the tensors tell
            w[q + "b"] = n((H, E), 1.5 / math.sqrt(E))
            w[q + "a1"], w[q + "a2"] = n((ra, E), 1.0 / math.sqrt(E)), n((H * N, ra), 1.0 / math.sqrt(ra))
            w[q + "dt_bias"] = n(H * N, 1.0, -1.0)
            w[q + "A_log"] = n(H, 0.7, -0.5)
            w[q + "g1"], w[q + "g2"] = n((rg, E), 1.0 / math.sqrt(E)), n((H * P, rg), 1.5 / math.sqrt(rg))
            w[q + "norm"] = n(P, 0.2, 1.0)
            w[q + "o"] = n((E, H * P), 0.7 / math.sqrt(H * P))
            w[q + "out"] = n(E, 0.1, 1.0)
        if lc["mlp"] is not None:
            F = lc["mlp"]["ff"]
            w[p + "mlp.up"] = n((F, E), 1.2 / math.sqrt(E))
            w[p + "mlp.down"] = n((E, F), 1.0 / math.sqrt(F))
            w[p + "mlp.act"] = helpers.bf16_round(np.array([0.75, 0.5, -0.25, 0.125]) + 0.1 * rng.standard_normal(4))
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
    cfg, w = pm.read_model(model_dir)
    return {r: pm.forward(cfg, w, toks) for r, toks in reqs.items()}


def random_config(rng, big):
    """A configuration drawn at random: two to six layers of either kind in any order, with sizes that the matrix-core
    kernels take (``big``) or that none of them takes."""
    def pick(*xs):
        return xs[int(rng.integers(0, len(xs)))]
    width = pick(128, 256, 384) if big else pick(24, 40, 56, 72, 100)
    layers = []
    for _ in range(int(rng.integers(2, 7))):
        if rng.random() < 0.45:
            mix = mlstm(pick(1, 2, 3, 4), pick(32, 64, 128) if big else pick(5, 8, 20), pick(32, 64, 96) if big else pick(4, 12, 30),
                        pick(1.0, 8.0, 15.0, 40.0))
        else:
            G = pick(1, 2, 4)
            D = pick(32, 64, 128) if big else pick(6, 10, 16, 24)
            lt = left(G * pick(1, 2, 3), G, D, D if big else pick(D, 4, 14), pick(1, 2, 3, 4), scale=pick(None, 0.2, 0.05))
            G = pick(1, 2, 3)
            rt = right(G * pick(1, 2), G, pick(32, 64, 128) if big else pick(3, 8, 17, 24), pick(16, 32, 64) if big else pick(4, 5, 12, 20),
                       pick(1, 2, 3, 4))
            mix = parallel(lt, rt)
        layers.append(layer(mix, None if rng.random() < 0.4 else pick(32, 64, 96, 48) if big else pick(4, 10, 24)))
    return config(int(rng.integers(50, 400)), width, layers, eps=pick(1e-5, 1e-6), embedding_scale=pick(1.0, 4.0, math.sqrt(width)),
                  logit_scale=pick(1.0, 0.5, 2.0))
