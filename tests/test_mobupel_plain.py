"""The plain implementation of the Mobupel design (tests/plain_mobupel.py) held against library routines, second
derivations and special cases, and the configuration reader and plan of the package. All on the CPU."""
import copy
import math

import numpy as np
import pytest
import torch

import mobupel_helpers as mh
import plain_mobupel as pm


def test_norm_has_eps_inside_the_root():
    assert np.allclose(pm.rms_norm(np.zeros((1, 4)) + 3.0, np.ones(4), 16.0), 3.0 / 5.0)
    assert np.allclose(pm.rms_div(np.array([[3.0, -4.0]]), 0.0), np.array([[3.0, -4.0]]) / math.sqrt(12.5))


def test_position_vector():
    s = pm.sinusoid([0, 1, 7], 6)
    assert np.allclose(s[0], [0, 1, 0, 1, 0, 1])
    for i in range(3):
        a = 7.0 * 10000.0 ** (-2.0 * i / 6)
        assert np.allclose(s[2, 2 * i:2 * i + 2], [math.sin(a), math.cos(a)])
    assert pm.sinusoid([3], 5).shape == (1, 5)                 # an odd width ends on a sine


def test_short_convolution_against_the_library():
    rng = np.random.default_rng(1)
    u, taps = rng.standard_normal((9, 3)), rng.standard_normal((3, 4))
    got = pm.causal_conv(u, taps)
    for c in range(3):
        assert np.allclose(got[:, c], np.convolve(u[:, c], taps[c, ::-1])[:9])          # the last tap is the current token's
    assert np.allclose(got[0], taps[:, -1] * u[0])                                         # zeros before the start
    assert np.allclose(pm.causal_conv(u, taps[:, :1]), u * taps[:, 0])                     # one tap: a factor a channel


def test_polynomial_activation():
    rng = np.random.default_rng(2)
    z = rng.standard_normal((4, 12))
    coef = np.array([0.5, -1.5, 2.0, 0.25])
    got = pm.poly_norm(z, coef, 0.0)
    # without eps every term is invariant under the row's scale up to sign
    assert np.allclose(pm.poly_norm(3.0 * z, coef, 0.0), got)
    want = sum(c * z ** p / np.sqrt((z ** (2 * p)).mean(-1, keepdims=True)) for c, p in zip(coef[:3], (1, 2, 3))) + coef[3]
    assert np.allclose(got, want)
    assert np.allclose(pm.poly_norm(np.zeros((1, 5)), coef, 1e-6), coef[3])


def test_matrix_memory_against_its_sum_form():
    """Without the running maximum: S~_t = sum over s <= t of exp(i_s + sum of f after s up to t) k_s v_s^T and n~_t alike;
    the stabilised S and n are these times exp(-m_t), so o_t = S~_t^T q / (max(|n~_t . q|, 1) + 1e-6 exp(m_t)), with
    m_t = max(f_t + m_(t-1), i_t) from m_0 = 0."""
    rng = np.random.default_rng(3)
    T, H, D, P = 12, 2, 3, 4
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, H, D)), rng.standard_normal((T, H, P))
    log_i, log_f = rng.standard_normal((T, H)) * 2.0, -rng.random((T, H)) * 1.5
    log_i[:3] = -4.0                                                      # the start's m = 0 stays the maximum for a while
    got = pm.mlstm_scan(q, k, v, log_i, log_f)
    for h in range(H):
        m = 0.0
        for t in range(T):
            m = max(log_f[t, h] + m, log_i[t, h])
            S, n = np.zeros((D, P)), np.zeros(D)
            for s in range(t + 1):
                a = math.exp(log_i[s, h] + log_f[s + 1:t + 1, h].sum())
                S += a * np.outer(k[s, h], v[s, h])
                n += a * k[s, h]
            want = S.T @ q[t, h] / (max(abs(n @ q[t, h]), 1.0) + 1e-6 * math.exp(m))
            assert np.allclose(got[t, h], want)
    # m_0 = 0: a first token whose input gate is far below 0 is written with the weight exp(i), where a maximum
    # that began below every gate would give it the weight 1
    o = pm.mlstm_scan(q[:1], k[:1], v[:1], np.full((1, H), -5.0), np.full((1, H), -0.1))
    for h in range(H):
        assert np.allclose(o[0, h], math.exp(-5.0) * (k[0, h] @ q[0, h]) * v[0, h] / (max(math.exp(-5.0) * abs(k[0, h] @ q[0, h]), 1.0) + 1e-6))


def test_gates_are_capped():
    z = np.array([-1e3, -2.0, 0.0, 2.0, 1e3])
    assert np.allclose(pm.soft_cap(z, 15.0), [-15.0, 15.0 * math.tanh(-2.0 / 15.0), 0.0, 15.0 * math.tanh(2.0 / 15.0), 15.0])
    assert np.allclose(pm.log_sigmoid(np.array([-800.0, 0.0, 800.0])), [-800.0, -math.log(2.0), 0.0])
    assert np.allclose(pm.softplus(np.array([-800.0, 0.0, 900.0])), [0.0, math.log(2.0), 900.0])


def test_attention_with_an_identity_mix_is_the_library_attention():
    rng = np.random.default_rng(4)
    T, H, G, D, P = 9, 4, 2, 6, 5
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, G, D)), rng.standard_normal((T, G, P))
    got = pm.talking_attention(q, k, v, 0.7, np.eye(H))
    tq = torch.from_numpy(q).permute(1, 0, 2)
    tk = torch.from_numpy(k).permute(1, 0, 2).repeat_interleave(H // G, 0)
    tv = torch.from_numpy(v).permute(1, 0, 2).repeat_interleave(H // G, 0)
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True, scale=0.7).permute(1, 0, 2).numpy()
    assert np.allclose(got, want, atol=1e-12)


def test_mixed_heads_apply_other_heads_weights_to_their_own_values():
    """out_h = sum_g talk[h, g] (weights_g applied to the values of h's group): by the library's attention with every
    head's queries and keys once for every group of values."""
    rng = np.random.default_rng(5)
    T, H, G, D, P = 7, 6, 3, 4, 5
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, G, D)), rng.standard_normal((T, G, P))
    talk = rng.standard_normal((H, H))
    got = pm.talking_attention(q, k, v, 0.3, talk)
    per = H // G
    tq = torch.from_numpy(q).permute(1, 0, 2)
    tk = torch.from_numpy(k).permute(1, 0, 2).repeat_interleave(per, 0)
    on_group = []                                                # [group of the values][head whose weights][T, P]
    for c in range(G):
        tv = torch.from_numpy(v[:, c]).unsqueeze(0).expand(H, T, P)
        on_group.append(torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True, scale=0.3).numpy())
    for h in range(H):
        want = sum(talk[h, g] * on_group[h // per][g] for g in range(H))
        assert np.allclose(got[:, h], want, atol=1e-12)
    # rows of the mix that do not sum to one, negative entries: nothing renormalises
    assert np.allclose(pm.talking_attention(q, k, v, 0.3, -2.0 * np.eye(H)), -2.0 * pm.talking_attention(q, k, v, 0.3, np.eye(H)))


def test_delta_rule_stores_a_value_at_its_key():
    """With strength 1 and no decay, reading with a unit key straight after its write gives its value back, whatever the
    state held; orthogonal keys do not disturb one another; a decay of zero on every row forgets everything before."""
    rng = np.random.default_rng(6)
    T, H, G, N, P = 6, 2, 1, 7, 3
    k = np.linalg.qr(rng.standard_normal((N, N)))[0][:T].reshape(T, 1, N)                  # orthonormal keys, one group
    v = rng.standard_normal((T, H, P))
    one, ones = np.ones((T, H)), np.ones((T, H, N))
    o = pm.delta_scan(k, k, v, one, ones)
    assert np.allclose(o, v)
    q = np.broadcast_to(k[0], (T, 1, N))
    assert np.allclose(pm.delta_scan(q, k, v, one, ones), np.broadcast_to(v[0], (T, H, P)))   # the first write stays readable
    # a second write at the same key with strength b moves the stored value by b of the way
    k2 = np.broadcast_to(k[0], (T, 1, N))
    b = np.full((T, H), 0.25)
    b[0] = 1.0
    o = pm.delta_scan(k2, k2, v, b, ones)
    want = v[0].copy()
    for t in range(1, T):
        want = want + 0.25 * (v[t] - want)
        assert np.allclose(o[t], want)
    # decays act before the write and per key channel: zero on all rows leaves only the token's own write
    o = pm.delta_scan(k2, k2, v, b, np.zeros((T, H, N)))
    assert np.allclose(o, b[:, :, None] * v)
    # a decay on the rows of one key channel only: S's other rows keep their content
    e = np.eye(N)[[0, 1, 0]].reshape(3, 1, N)
    d = np.ones((3, 1, N))
    d[2, 0, 1] = 0.0
    vv = rng.standard_normal((3, 1, P))
    o = pm.delta_scan(np.eye(N)[[0, 1, 1]].reshape(3, 1, N), e, vv, np.array([[1.0], [1.0], [0.0]]), d)
    assert np.allclose(o[2], 0.0) and np.allclose(o[1], vv[1])


def test_unit_vectors():
    x = np.array([[3.0, 4.0]])
    assert np.allclose(pm.unit(x, 0.0), [[0.6, 0.8]])
    assert np.allclose(pm.unit(np.zeros((1, 2))), 0.0)
    assert np.allclose(pm.unit(x), x / math.sqrt(25.0 + 1e-6))


@pytest.fixture(scope="module")
def small():
    cfg = mh.SMALL
    return cfg, {k: np.asarray(v, np.float64) for k, v in mh.make_weights(cfg, 3).items()}


def test_a_prefix_has_the_logits_of_the_whole(small):
    cfg, w = small
    toks = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 30)]
    whole = pm.forward(cfg, w, toks)
    assert np.allclose(pm.forward(cfg, w, toks[:13]), whole[:13], atol=1e-9)
    assert np.all(np.isfinite(whole))


def test_closed_gates_leave_the_embedding(small):
    """The sublayers' gates far below zero: every result is multiplied by nearly zero, and the norm after it, whose eps
    is inside the root, keeps it small; the logits are those of the embedding with its position vector."""
    cfg, w = small
    w = dict(w)
    for name in list(w):
        if name.endswith(".b") and ".rg" in name:
            w[name] = np.full_like(w[name], -80.0)
            w[name[:-2]] = np.zeros_like(w[name[:-2]])
    toks = [5, 9, 77, 9]
    x = w["embed"][toks] * cfg["embedding"]["scale"] + pm.sinusoid(range(4), cfg["width"])
    want = pm.rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T * cfg["logit_scale"]
    assert np.allclose(pm.forward(cfg, w, toks), want, atol=1e-6)
    assert not np.allclose(want[1], want[3])                            # the same token at another position


def test_each_side_is_normed_before_half_their_sum(small):
    cfg, w = small
    rng = np.random.default_rng(8)
    h = rng.standard_normal((5, cfg["width"]))
    m, eps = cfg["layers"][1]["mixer"], cfg["norm"]["eps"]
    both = pm.parallel_mixer(h, w, "l1.mix.", m, eps)
    w2 = dict(w)
    w2["l1.mix.right.o"] = w["l1.mix.right.o"] * 7.0                     # a side's scale does not pass its norm
    assert np.allclose(pm.parallel_mixer(h, w2, "l1.mix.", m, eps), both, atol=1e-4)
    lt = pm.rms_norm(pm.left_attention(h, w, "l1.mix.left.", m["left"], eps), w["l1.mix.left.out"], eps)
    rt = pm.rms_norm(pm.right_delta(h, w, "l1.mix.right.", m["right"], eps), w["l1.mix.right.out"], eps)
    assert np.allclose(both, 0.5 * (lt + rt))


# ---- the package's configuration reader and plan ----------------------------------------------------------------

def test_configuration_and_plan():
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.kernels.ops import Ops
    from hf_cpu_amd.parts.base import FixedState, PagedKV
    for name, cfg in mh.CONFIGS.items():
        c = config_from_dict(cfg)
        assert c.width == cfg["width"] and len(c.layers) == len(cfg["layers"]) and c.to_dict() == cfg
        model = hf_cpu_amd.Model.from_config(c)
        declared = {s.name: tuple(s.shape) for s in model.param_specs() if not s.optional}
        made = {k: tuple(np.shape(v)) for k, v in mh.make_weights(cfg, 0).items()}
        assert set(declared) == set(made)
        for k, shape in declared.items():              # (0: a size that only the tensor tells)
            assert len(shape) == len(made[k]) and all(a in (0, b) for a, b in zip(shape, made[k])), k
        assert len(model.cache_needs()) == sum(1 if lc["type"] == "mlstm" else 2 + (lc["mixer"]["left"]["conv"] > 1) for lc in cfg["layers"])
        for lc, lay in zip(cfg["layers"], model.layers):
            m, need = lc["mixer"], dict(lay.cache_parts())["mixer"].cache_need()
            if lc["type"] == "mlstm":
                assert need == FixedState(Ops.scan_state_floats(m["heads"], m["dim"], m["vdim"], normalizer=True))
                assert need.n_floats >= m["heads"] * (m["dim"] * (m["vdim"] + 1) + 1)
            else:
                lt, rt = m["left"], m["right"]
                channels = 2 * rt["kv_heads"] * rt["dim"] + rt["heads"] * rt["vdim"]
                assert need["right"] == FixedState(Ops.scan_state_floats(rt["heads"], rt["dim"], rt["vdim"]) + (rt["conv"] - 1) * channels)
                kv = need["left"]["kv"] if isinstance(need["left"], dict) else need["left"]
                assert kv == PagedKV(lt["kv_heads"] * lt["dim"], lt["kv_heads"] * lt["vdim"])
                if lt["conv"] > 1:
                    assert need["left"]["conv"] == FixedState((lt["conv"] - 1) * (lt["heads"] * lt["dim"] + lt["kv_heads"] * (lt["dim"] + lt["vdim"])))


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="conv"), "not supported"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=4), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mlp"].update(kind="moe"), "not supported"),
    (lambda c: c["layers"][0]["mixer"].pop("gate_cap"), "gate_cap"),
    (lambda c: c["layers"][4]["mixer"].pop("left"), "left"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.pop("logit_scale"), "logit_scale"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(conv=9), "conv"),
])
def test_configuration_errors_name_what_is_wrong(change, word):
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.status import EngineError
    cfg = copy.deepcopy(mh.SMALL)
    change(cfg)
    with pytest.raises(EngineError) as e:
        config_from_dict(cfg)
    assert word in str(e.value.msg)
