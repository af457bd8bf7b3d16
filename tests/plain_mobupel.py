"""The plain implementation of the Mobupel design: whole sequences, float64 numpy, one function a mechanism.

No cache, no batching, no kernels, and no code shared with the package. The engine is compared with this.

The stream starts as ``embed[token] * scale`` plus a sinusoidal position vector. A layer is
``x <- x + post1(gate1(h) * mixer(h))`` with ``h = pre1(x)``, then the same around the feed-forward where the layer has
one: RMS norms before and after each sublayer, and a sigmoid gate computed from the sublayer's input that multiplies
the sublayer's result before the second norm. Two mixers:

* ``mlstm``: a matrix memory per head with exponential input gates and sigmoid forget gates (both soft-capped), kept
  stable by a running maximum of the gates' logarithms; a normaliser vector beside the matrix; the read-out is normed
  head by head, gated and projected.
* ``parallel``: two mixers side by side on the same input, each result RMS-normed over the width, half their sum.
  Left: softmax attention with grouped heads, a short causal convolution on q, k and v, per-head RMS norm of queries and
  keys, no positions, attention weights mixed across heads after the softmax, a sigmoid output gate. Right: the gated
  delta rule: q, k, v through a short convolution and silu, unit-length q and k, a decay per key channel, a write
  strength per head, and a state that is corrected towards ``v`` along ``k``.

The feed-forward is ``Wdown act(Wup h)`` with a polynomial activation of normed powers.
"""
import numpy as np

from plain import read_model          # noqa: F401  (the container reader is the same for every design)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w


def rms_div(x, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def sinusoid(positions, width, base=10000.0):
    """[T, width]: entry 2i is sin(p base^(-2i / width)), entry 2i + 1 the cosine of the same angle."""
    out = np.zeros((len(positions), width))
    p = np.asarray(positions, dtype=np.float64)[:, None]
    i = np.arange((width + 1) // 2, dtype=np.float64)[None, :]
    ang = p * base ** (-2.0 * i / width)
    out[:, 0::2] = np.sin(ang)[:, :out[:, 0::2].shape[1]]
    out[:, 1::2] = np.cos(ang)[:, :out[:, 1::2].shape[1]]
    return out


def causal_conv(u, taps):
    """u: [T, C], taps: [C, K]. out[t] = sum_j taps[:, j] u[t - (K - 1) + j]; zeros before t = 0."""
    T, C = u.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), u], axis=0)
    out = np.zeros((T, C))
    for j in range(K):
        out += padded[j:j + T] * taps[:, j]
    return out


def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e, N dividing a row by its root mean square."""
    a, b, c, e = coef
    return a * rms_div(z, eps) + b * rms_div(z ** 2, eps) + c * rms_div(z ** 3, eps) + e


def feed_forward(h, w, p, eps):
    return poly_norm(h @ w[p + "up"].T, w[p + "act"], eps) @ w[p + "down"].T


def soft_cap(z, cap):
    return cap * np.tanh(z / cap)


def mlstm_scan(q, k, v, log_i, log_f):
    """q, k: [T, H, D] (q already scaled), v: [T, H, P], log_i, log_f: [T, H]. Per head, with m_0 = 0, S_0 = 0, n_0 = 0:
    m_t = max(log_f + m_(t-1), log_i); S_t = exp(log_f + m_(t-1) - m_t) S_(t-1) + exp(log_i - m_t) k v^T; n_t alike with k;
    o_t = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)."""
    T, H, D = q.shape
    P = v.shape[2]
    o = np.zeros((T, H, P))
    for h in range(H):
        S, n, m = np.zeros((D, P)), np.zeros(D), 0.0
        for t in range(T):
            m_new = max(log_f[t, h] + m, log_i[t, h])
            a, b = np.exp(log_f[t, h] + m - m_new), np.exp(log_i[t, h] - m_new)
            S = a * S + b * np.outer(k[t, h], v[t, h])
            n = a * n + b * k[t, h]
            m = m_new
            o[t, h] = S.T @ q[t, h] / (max(abs(n @ q[t, h]), np.exp(-m)) + 1e-6)
    return o


def mlstm(h, w, p, m, eps):
    """The whole mixer on the normed stream h: [T, width]; w: tensors by name, p: their prefix, m: the mixer's sizes."""
    T = h.shape[0]
    H, D, P, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, P)
    log_i = soft_cap(h @ w[p + "i"].T + w[p + "i.b"], cap)
    log_f = log_sigmoid(soft_cap(h @ w[p + "f"].T + w[p + "f.b"], cap))
    o = rms_div(mlstm_scan(q, k, v, log_i, log_f), eps).reshape(T, H * P)
    return (o * w[p + "norm"] * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def talking_attention(q, k, v, scale, talk):
    """q: [T, H, D], k: [T, G, D], v: [T, G, P]; causal softmax of (q . k) scale per head; the heads' weights are then
    mixed, weight_h <- sum_g talk[h, g] weight_g, and head h applies its mixed weights to the values of its own group."""
    T, H, D = q.shape
    G = k.shape[1]
    per = H // G
    w = np.zeros((H, T, T))
    mask = np.tril(np.ones((T, T), dtype=bool))
    for h in range(H):
        s = (q[:, h] @ k[:, h // per].T) * scale
        s = np.where(mask, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        e = np.exp(s)
        w[h] = e / e.sum(axis=1, keepdims=True)
    mixed = np.einsum("hg,gij->hij", talk, w)
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        out[:, h] = mixed[h] @ v[:, h // per]
    return out


def left_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv(h @ w[p + "q"].T, w[p + "q.conv"]).reshape(T, H, D)
    k = causal_conv(h @ w[p + "k"].T, w[p + "k.conv"]).reshape(T, G, D)
    v = causal_conv(h @ w[p + "v"].T, w[p + "v.conv"]).reshape(T, G, P)
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)
    att = talking_attention(q, k, v, m["scale"], w[p + "talk"]).reshape(T, H * P)
    return (att * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def delta_scan(q, k, v, beta, decay):
    """q, k: [T, G, N], v: [T, H, P], beta: [T, H], decay: [T, H, N]; head h reads q and k of head h // (H / G). Per head:
    S <- decay_t[:, None] * S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t."""
    T, H, P = v.shape
    G, N = q.shape[1], q.shape[2]
    per = H // G
    o = np.zeros((T, H, P))
    for h in range(H):
        S = np.zeros((N, P))
        g = h // per
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
            S = S + np.outer(k[t, g], u)
            o[t, h] = S.T @ q[t, g]
    return o


def unit(x, eps=1e-6):
    return x / np.sqrt((x * x).sum(axis=-1, keepdims=True) + eps)


def right_delta(h, w, p, m, eps):
    T = h.shape[0]
    H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, N)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, N)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, P)
    q, k = unit(q) * N ** -0.5, unit(k)
    beta = sigmoid(h @ w[p + "b"].T)
    rate = np.exp(w[p + "A_log"])[None, :, None]
    decay = np.exp(-rate * softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, N))
    o = rms_norm(delta_scan(q, k, v, beta, decay), w[p + "norm"], eps).reshape(T, H * P)
    return (o * sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T)) @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    left = rms_norm(left_attention(h, w, p + "left.", m["left"], eps), w[p + "left.out"], eps)
    right = rms_norm(right_delta(h, w, p + "right.", m["right"], eps), w[p + "right.out"], eps)
    return 0.5 * (left + right)


def sublayer(x, w, p, which, eps, fn):
    """x + post(gate(h) * fn(h)) with h = pre(x); ``which`` is "1" for the mixer, "2" for the feed-forward."""
    h = rms_norm(x, w[p + "norm" + which], eps)
    y = fn(h) * sigmoid(h @ w[p + "rg" + which].T + w[p + "rg" + which + ".b"])
    return x + rms_norm(y, w[p + "norm" + which + "b"], eps)


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence. ``layers_out``: a list that receives the stream after every layer."""
    w = {n: np.asarray(t, dtype=np.float64) for n, t in w.items()}
    eps, E = cfg["norm"]["eps"], cfg["width"]
    tokens = np.asarray(tokens)
    x = w["embed"][tokens] * cfg["embedding"]["scale"] + sinusoid(np.arange(len(tokens)), E)
    for l, lc in enumerate(cfg["layers"]):
        p = f"l{l}."
        mix = {"mlstm": mlstm, "parallel": parallel_mixer}[lc["type"]]
        x = sublayer(x, w, p, "1", eps, lambda h: mix(h, w, p + "mix.", lc["mixer"], eps))
        if lc.get("mlp") is not None:
            x = sublayer(x, w, p, "2", eps, lambda h: feed_forward(h, w, p + "mlp.", eps))
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T * cfg["logit_scale"]
