"""The plain implementation of the Gitasun design: whole sequences, float64 numpy, one function a mechanism.

No cache, no batching, no kernels, and no code shared with the package. The engine is compared with this.

The stream starts as ``embed[token] * scale``. A layer is ``x <- x + m * ls1 * mixer(norm1(x))``, then
``x <- x + m * ls2 * ff(norm2(x))`` where the layer has a feed-forward: ``m`` one number for the whole model, ``ls1`` and ``ls2``
a vector each, the norms RMS norms whose weight is a single number. Three mixers:

* ``latent_attention``: causal softmax attention whose queries come through a normed latent and whose keys and values are
  expanded from one normed latent a token; a head's query and key have an unrotated part and a rotated part, the rotated
  key part being one vector a token that all heads share; a sigmoid gate on the heads before the output projection.
* ``hgrn2``: a linear recurrence per head whose forget gate (bounded below) decays the rows of the state and whose
  complement is the key that writes the value.
* ``parallel``: the weighted sum of two mixers on the same input. Left: causal attention with grouped heads, biases,
  rotation with rescaled frequencies, soft-capped scores and sigmoid weights (no softmax), a sigmoid gate on the heads.
  Right: gated linear attention with a decay per key channel from a low-rank projection, a per-head norm and a silu gate.

The feed-forward is dense (``Wdown gelu_tanh(Wup h)``) or a mixture of gated experts with a shared expert.
"""
import math

import numpy as np

from plain import read_model          # noqa: F401  (the container reader is the same for every design)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w a vector or one number)."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i / dims) for i < dims / 2. ``scaling`` (factor, low, high, original): with the wavelength l = 2 pi / f, f
    stays where l < original / high, becomes f / factor where l > original / low, and in between is the blend
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    f = base ** (-2.0 * np.arange(dims // 2, dtype=np.float64) / dims)
    if scaling is None:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = np.empty_like(f)
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            out[i] = fi
        elif wavelength > original / low:
            out[i] = fi / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate(x, positions, freqs):
    """x: [T, ..., n] with n >= 2 len(freqs): dimension i of the first 2 len(freqs) is paired with i + len(freqs); the pair
    (u, v) at position p becomes (u cos a - v sin a, v cos a + u sin a), a = p f_i. The rest passes unchanged."""
    half = len(freqs)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    cos, sin = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:2 * half]
    out = x.copy()
    out[..., :half] = u * cos - v * sin
    out[..., half:2 * half] = v * cos + u * sin
    return out


def causal_softmax_attention(q, k, v, scale):
    """q: [T, H, D], k: [T, H, D], v: [T, H, Dv] -> [T, H, Dv]; position i sees every j <= i."""
    T = q.shape[0]
    s = np.einsum("ihd,jhd->hij", q, k) * scale
    s = np.where(np.tril(np.ones((T, T), dtype=bool))[None], s, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("hij,jhd->ihd", p, v)


def latent_attention(h, w, p, m, eps, positions):
    """``m``: heads, dim, rot_dim, vdim, kv_rank, scale, rot = {base, dims}."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freqs = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(T, H, D + R)
    q_flat, q_rot = q[..., :D], rotate(q[..., D:], positions, freqs)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :C], w[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, C:], positions, freqs)                     # one vector a token, for all heads
    k_flat = (c @ w[p + "uk"].T).reshape(T, H, D)
    v = (c @ w[p + "uv"].T).reshape(T, H, Dv)
    qq = np.concatenate([q_flat, q_rot], axis=-1)
    kk = np.concatenate([k_flat, np.broadcast_to(k_rot[:, None, :], (T, H, R))], axis=-1)
    o = causal_softmax_attention(qq, kk, v, m["scale"]).reshape(T, H * Dv)
    return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def channel_decay_recurrence(q, k, v, a):
    """q, k, a: [T, H, D]; v: [T, H, Dv]. Per head S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t; S_0 = 0."""
    T, H, D = q.shape
    S = np.zeros((H, D, v.shape[2]))
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        S = a[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = np.einsum("hdv,hd->hv", S, q[t])
    return out


def hgrn2(h, w, p, m, eps):
    """``m``: heads, dim, vdim."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, Dv)
    lower = w[p + "lower"]
    f = (lower + (1.0 - lower) * sigmoid(h @ w[p + "f"].T + w[p + "f.b"])).reshape(T, H, D)
    o = channel_decay_recurrence(q, 1.0 - f, v, f)
    return rms_norm(o, w[p + "norm"], eps).reshape(T, H * Dv) @ w[p + "o"].T


def sigmoid_attention(h, w, p, m, positions):
    """The left side of ``parallel``. ``m``: heads, kv_heads, dim, vdim, scale, softcap, rot = {base, dims, scaling}."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    freqs = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q = rotate((h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D), positions, freqs)
    k = rotate((h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D), positions, freqs)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, Dv)
    group = np.arange(H) // (H // G)
    s = np.einsum("ihd,jhd->hij", q, k[:, group]) * m["scale"]
    cap = m.get("softcap")
    if cap:
        s = cap * np.tanh(s / cap)
    weights = sigmoid(s + w[p + "pb"][:, None, None]) * np.tril(np.ones((T, T)))[None]
    o = np.einsum("hij,jhd->ihd", weights, v[:, group]).reshape(T, H * Dv)
    return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def gated_linear_attention(h, w, p, m, eps):
    """The right side of ``parallel``. ``m``: heads, dim, vdim, tau."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, Dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, D)
    o = channel_decay_recurrence(q, k, v, alpha)
    o = rms_norm(o, w[p + "norm"], eps).reshape(T, H * Dv)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel(h, w, p, m, eps, positions):
    return m["left_scale"] * sigmoid_attention(h, w, p + "left.", m["left"], positions) \
        + m["right_scale"] * gated_linear_attention(h, w, p + "right.", m["right"], eps)


def gated_unit(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, top):
    """(ids [T, top], weights [T, top]): the ``top`` largest logits (the lower index among equals), softmax over them alone."""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    ids = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(z, ids, axis=-1)
    e = np.exp(chosen - chosen.max(axis=-1, keepdims=True))
    return ids, e / e.sum(axis=-1, keepdims=True)


def feed_forward(h, w, p, f):
    if f["kind"] == "dense":
        return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T
    ids, weights = route(h, w, p, f["router"]["top"])
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, c in zip(ids[t], weights[t]):
            out[t] += c * gated_unit(h[t:t + 1], w, f"{p}e{e}.")[0]
    if f.get("shared") is not None:
        out += gated_unit(h, w, p + "shared.")
    return out


def mixer(kind, h, w, p, m, eps, positions):
    if kind == "latent_attention":
        return latent_attention(h, w, p, m, eps, positions)
    if kind == "hgrn2":
        return hgrn2(h, w, p, m, eps)
    if kind == "parallel":
        return parallel(h, w, p, m, eps, positions)
    raise ValueError(f"unknown mixer '{kind}'")


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence. ``layers_out``: a list that receives the stream after every layer."""
    w = {k: np.asarray(v, dtype=np.float64) for k, v in w.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    positions = np.arange(len(tokens))
    x = w["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, w[p + "norm1"], eps)
        x = x + mult * w[p + "ls1"] * mixer(lc["type"], h, w, p + "mix.", lc["mixer"], eps, positions)
        if lc.get("mlp") is not None:
            h = rms_norm(x, w[p + "norm2"], eps)
            x = x + mult * w[p + "ls2"] * feed_forward(h, w, p + "mlp.", lc["mlp"])
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
