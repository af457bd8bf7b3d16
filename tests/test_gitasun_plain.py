"""The plain implementation of the Gitasun design (tests/plain_gitasun.py) held against second derivations and special
cases, and the configuration reader and plan of the package. All on the CPU."""
import copy
import math

import numpy as np
import pytest

import gitasun_helpers as gh
import plain_gitasun as pg


def test_norm_has_eps_inside_the_root_and_takes_one_number():
    assert np.allclose(pg.rms_norm(np.zeros((1, 4)) + 3.0, 2.0, 16.0), 2.0 * 3.0 / 5.0)
    assert np.allclose(pg.rms_norm(np.array([[3.0, -4.0]]), np.array([1.0, 2.0]), 0.0), np.array([[3.0, -8.0]]) / math.sqrt(12.5))


def test_tanh_gelu():
    z = np.array([-3.0, -0.5, 0.0, 0.7, 4.0])
    want = [0.5 * x * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3))) for x in z]
    assert np.allclose(pg.gelu_tanh(z), want)
    assert abs(pg.gelu_tanh(np.array([10.0]))[0] - 10.0) < 1e-9 and abs(pg.gelu_tanh(np.array([-10.0]))[0]) < 1e-9


def test_rescaled_frequencies():
    base, dims = 30000.0, 40
    f = pg.rotary_frequencies(dims, base)
    assert np.allclose(f, [base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = dict(factor=6.0, low=1.0, high=3.0, original=256)
    g = pg.rotary_frequencies(dims, base, sc)
    wl = 2.0 * math.pi / f
    short, long_ = 256 / 3.0, 256.0
    assert np.array_equal(g[wl < short], f[wl < short]) and np.allclose(g[wl > long_], f[wl > long_] / 6.0)
    mid = (wl >= short) & (wl <= long_)
    assert mid.any() and (wl < short).any() and (wl > long_).any()
    assert np.all(g[mid] <= f[mid]) and np.all(g[mid] >= f[mid] / 6.0)
    # the blend meets both ends: at l = original / high it is f, at l = original / low it is f / factor
    for l_, want in ((short, 1.0), (long_, 1.0 / 6.0)):
        s = (256.0 / l_ - 1.0) / 2.0
        assert math.isclose((1.0 - s) / 6.0 + s, want)
    assert np.allclose(pg.rotary_frequencies(dims, base, dict(sc, factor=1.0)), f, rtol=1e-14)


def test_rotation_pairs_i_with_i_plus_half_and_keeps_the_rest():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 3, 10))
    f = pg.rotary_frequencies(6, 100.0)
    y = pg.rotate(x, [0, 1, 2, 9, 400], f)
    assert np.array_equal(y[0], x[0]) and np.array_equal(y[..., 6:], x[..., 6:])
    a = 9 * f[1]
    assert np.allclose(y[3, :, 1], x[3, :, 1] * math.cos(a) - x[3, :, 4] * math.sin(a))
    assert np.allclose(y[3, :, 4], x[3, :, 4] * math.cos(a) + x[3, :, 1] * math.sin(a))
    # a score of rotated vectors depends on the distance alone
    q, k = rng.standard_normal((1, 6)), rng.standard_normal((1, 6))
    d1 = (pg.rotate(q, [17], f) * pg.rotate(k, [12], f)).sum()
    d2 = (pg.rotate(q, [105], f) * pg.rotate(k, [100], f)).sum()
    assert math.isclose(d1, d2, rel_tol=1e-9)


def test_recurrence_against_its_sum_form():
    """o_t = sum over s <= t of ((prod of a after s up to t) * k_s . q_t) v_s."""
    rng = np.random.default_rng(1)
    T, H, D, P = 9, 2, 3, 4
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, H, D)), rng.standard_normal((T, H, P))
    a = rng.uniform(0.1, 1.0, (T, H, D))
    got = pg.channel_decay_recurrence(q, k, v, a)
    for t in range(T):
        want = np.zeros((H, P))
        for s in range(t + 1):
            decay = np.prod(a[s + 1:t + 1], axis=0)
            want += ((decay * k[s] * q[t]).sum(-1))[:, None] * v[s]
        assert np.allclose(got[t], want)


def small_weights(cfg, seed=0):
    return {k: np.asarray(v, np.float64) for k, v in gh.make_weights(cfg, seed).items()}


def test_forget_gate_recurrence_special_cases():
    cfg = gh.config(20, 12, [gh.layer(gh.hgrn2(2, 3, 4), None)])
    w = small_weights(cfg)
    h = np.random.default_rng(2).standard_normal((6, 12))
    p, m = "l0.mix.", cfg["layers"][0]["mixer"]
    # a gate that never forgets never writes: the result is zero
    w2 = dict(w)
    w2[p + "f.b"] = w[p + "f.b"] + 1e4
    assert np.allclose(pg.hgrn2(h, w2, p, m, 1e-6), 0.0)
    # no lower bound and a gate that forgets everything: S_t = 1 v_t^T, o_t = sum(q_t) v_t, normed head by head
    w3 = dict(w)
    w3[p + "f.b"], w3[p + "lower"] = w[p + "f.b"] - 1e4, np.zeros(6)
    q = pg.silu(h @ w[p + "q"].T).reshape(6, 2, 3)
    v = (h @ w[p + "v"].T).reshape(6, 2, 4)
    want = pg.rms_norm(q.sum(-1, keepdims=True) * v, w[p + "norm"], 1e-6).reshape(6, 8) @ w[p + "o"].T
    assert np.allclose(pg.hgrn2(h, w3, p, m, 1e-6), want)
    # the lower bound is a bound: with the gate shut the decay is the bound itself
    w4 = dict(w3)
    w4[p + "lower"] = np.full(6, 0.25)
    f = 0.25
    S = np.zeros((2, 3, 4))
    out = []
    for t in range(6):
        S = f * S + (1 - f) * np.ones((2, 3, 1)) * v[t][:, None, :]
        out.append(np.einsum("hdv,hd->hv", S, q[t]))
    want = pg.rms_norm(np.array(out), w[p + "norm"], 1e-6).reshape(6, 8) @ w[p + "o"].T
    assert np.allclose(pg.hgrn2(h, w4, p, m, 1e-6), want)


def test_gated_linear_attention_without_decay_is_a_running_sum():
    cfg = gh.config(20, 12, [gh.layer(gh.parallel(gh.left(2, 1, 4, 4, 4), gh.right(2, 3, 4, 2.0)), None)])
    w = small_weights(cfg)
    h = np.random.default_rng(3).standard_normal((7, 12))
    p, m = "l0.mix.right.", cfg["layers"][0]["mixer"]["right"]
    w2 = dict(w)
    w2[p + "a2.b"] = w[p + "a2.b"] + 1e4                     # sigmoid -> 1: nothing decays
    q = (h @ w[p + "q"].T).reshape(7, 2, 3) / math.sqrt(3)
    k, v = (h @ w[p + "k"].T).reshape(7, 2, 3), (h @ w[p + "v"].T).reshape(7, 2, 4)
    scores = np.einsum("ihd,jhd->hij", q, k) * np.tril(np.ones((7, 7)))
    o = np.einsum("hij,jhv->ihv", scores, v)
    want = (pg.rms_norm(o, w[p + "norm"], 1e-6).reshape(7, 8) * pg.silu(h @ w[p + "g"].T)) @ w[p + "o"].T
    assert np.allclose(pg.gated_linear_attention(h, w2, p, m, 1e-6), want)
    # tau is a root of the sigmoid: with z = 0 the decay is 0.5^(1 / tau)
    w3 = dict(w)
    w3[p + "a2"], w3[p + "a2.b"] = np.zeros_like(w[p + "a2"]), np.zeros(6)
    a = np.full((7, 2, 3), 0.5 ** 0.5)
    o = pg.channel_decay_recurrence(q, k, v, a)
    want = (pg.rms_norm(o, w[p + "norm"], 1e-6).reshape(7, 8) * pg.silu(h @ w[p + "g"].T)) @ w[p + "o"].T
    assert np.allclose(pg.gated_linear_attention(h, w3, p, m, 1e-6), want)


def test_sigmoid_attention_special_cases():
    cfg = gh.config(20, 12, [gh.layer(gh.parallel(gh.left(4, 2, 6, 5, 4, softcap=2.0, scale=0.5), gh.right(1, 3, 4, 2.0)), None)])
    w = small_weights(cfg)
    rng = np.random.default_rng(4)
    h = rng.standard_normal((5, 12))
    p, m = "l0.mix.left.", cfg["layers"][0]["mixer"]["left"]
    pos = np.arange(5)
    got = pg.sigmoid_attention(h, w, p, m, pos)
    # the first token sees itself alone: one weight, sigmoid(capped score + the head's number), on its own value
    q = pg.rotate((h[:1] @ w[p + "q"].T + w[p + "q.b"]).reshape(1, 4, 6), [0], pg.rotary_frequencies(4, 10000.0))
    k = (h[:1] @ w[p + "k"].T + w[p + "k.b"]).reshape(1, 2, 6)
    v = (h[:1] @ w[p + "v"].T + w[p + "v.b"]).reshape(1, 2, 5)
    grp = np.array([0, 0, 1, 1])
    s = 2.0 * np.tanh((q[0] * k[0][grp]).sum(-1) * 0.5 / 2.0)
    o = (pg.sigmoid(s + w[p + "pb"])[:, None] * v[0][grp]).reshape(1, 20)
    assert np.allclose(got[:1], (o * pg.sigmoid(h[:1] @ w[p + "g"].T)) @ w[p + "o"].T)
    # the weights are not normalised: with numbers so large that every weight is 1, a head's result is the running sum of its values
    w2 = dict(w)
    w2[p + "pb"] = np.full(4, 1e4)
    vv = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(5, 2, 5)
    o = np.cumsum(vv, axis=0)[:, grp].reshape(5, 20)
    assert np.allclose(pg.sigmoid_attention(h, w2, p, m, pos), (o * pg.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T)
    # the cap bounds the scores: queries a thousand times larger change nothing once tanh is at its end
    w3, w4 = dict(w), dict(w)
    w3[p + "q"], w3[p + "q.b"] = w[p + "q"] * 1e3, w[p + "q.b"] * 1e3
    w4[p + "q"], w4[p + "q.b"] = w[p + "q"] * 1e6, w[p + "q.b"] * 1e6
    assert np.allclose(pg.sigmoid_attention(h, w3, p, m, pos), pg.sigmoid_attention(h, w4, p, m, pos), atol=1e-9)
    m2 = dict(m)
    del m2["softcap"]
    assert not np.allclose(pg.sigmoid_attention(h, w, p, m2, pos), got)


def test_latent_attention_against_the_form_that_keeps_latents_only():
    """Folding the keys' expansion into the queries and taking the values' out of the sum gives the same result: the score is
    (Wuk_h^T q_h) . c + q_rot . k_rot and the head's output Wuv_h (sum_j p_j c_j)."""
    cfg = gh.config(20, 16, [gh.layer(gh.latent(3, 4, 6, 5, 7, 9, base=30.0, rot_dims=4), None)])
    w = small_weights(cfg)
    rng = np.random.default_rng(5)
    T = 8
    h = rng.standard_normal((T, 16))
    p, m = "l0.mix.", cfg["layers"][0]["mixer"]
    pos = np.arange(T) + 3
    got = pg.latent_attention(h, w, p, m, 1e-6, pos)
    H, D, R, P, C = 3, 4, 6, 5, 7
    f = pg.rotary_frequencies(4, 30.0)
    cq = pg.rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], 1e-6)
    q = (cq @ w[p + "uq"].T).reshape(T, H, D + R)
    down = h @ w[p + "dkv"].T
    c = pg.rms_norm(down[:, :C], w[p + "dkv.norm"], 1e-6)
    k_rot = pg.rotate(down[:, C:], pos, f)
    out = np.zeros((T, H, P))
    for hd in range(H):
        q_lat = q[:, hd, :D] @ w[p + "uk"][hd * D:(hd + 1) * D]              # [T, C]
        q_rot = pg.rotate(q[:, hd, D:], pos, f)
        for i in range(T):
            s = (c[:i + 1] @ q_lat[i] + k_rot[:i + 1] @ q_rot[i]) * m["scale"]
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            out[i, hd] = w[p + "uv"][hd * P:(hd + 1) * P] @ (pr @ c[:i + 1])
    want = (out.reshape(T, H * P) * pg.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T
    assert np.allclose(got, want)


def test_router_and_experts():
    cfg = gh.config(20, 12, [gh.layer(gh.hgrn2(1, 3, 4), gh.moe(5, 2, 6, shared=4))])
    w = small_weights(cfg)
    h = np.random.default_rng(6).standard_normal((9, 12))
    p = "l0.mlp."
    ids, wts = pg.route(h, w, p, 2)
    z = h @ w[p + "router"].T + w[p + "router.b"]
    assert np.allclose(wts.sum(-1), 1.0)
    for t in range(9):
        order = np.argsort(-z[t])
        assert list(ids[t]) == list(order[:2])
        assert math.isclose(wts[t, 0] / wts[t, 1], math.exp(z[t, ids[t, 0]] - z[t, ids[t, 1]]), rel_tol=1e-9)
    # all experts chosen: the softmax over all logits weighs all experts; the shared expert is added unweighted
    f_all = gh.moe(5, 5, 6, shared=4)
    sm = np.exp(z - z.max(-1, keepdims=True))
    sm /= sm.sum(-1, keepdims=True)
    want = sum(sm[:, e:e + 1] * pg.gated_unit(h, w, f"{p}e{e}.") for e in range(5)) + pg.gated_unit(h, w, p + "shared.")
    assert np.allclose(pg.feed_forward(h, w, p, f_all), want)
    f_none = gh.moe(5, 5, 6)
    assert np.allclose(pg.feed_forward(h, w, p, f_none), want - pg.gated_unit(h, w, p + "shared."))
    one = gh.moe(5, 1, 6)
    got = pg.feed_forward(h, w, p, one)
    for t in range(9):
        assert np.allclose(got[t], pg.gated_unit(h[t:t + 1], w, f"{p}e{int(np.argmax(z[t]))}.")[0])      # a single choice weighs 1


def test_a_model_whose_branches_are_silenced_is_its_head():
    cfg = copy.deepcopy(gh.SMALL)
    w = small_weights(cfg, 3)
    toks = [5, 9, 130, 0, 77]
    for k in list(w):
        if k.endswith(".ls1") or k.endswith(".ls2"):
            w[k] = np.zeros_like(w[k])
    want = pg.rms_norm(w["embed"][toks] * 3.0, w["final.norm"], 1e-5) @ w["head"].T
    assert np.allclose(pg.forward(cfg, w, toks), want)
    # and the multiplier scales every branch: m = 0 does the same
    w = small_weights(cfg, 3)
    cfg["residual_mult"] = 0.0
    assert np.allclose(pg.forward(cfg, w, toks), want)


def test_a_position_does_not_depend_on_what_follows():
    cfg = gh.SMALL
    w = small_weights(cfg, 1)
    toks = [int(t) for t in np.random.default_rng(7).integers(0, cfg["vocab"], 14)]
    whole = pg.forward(cfg, w, toks)
    assert np.allclose(pg.forward(cfg, w, toks[:9]), whole[:9])


# ---- the package's reader and plan ------------------------------------------------------------------------------------

def test_configuration_reads_every_size_and_constant():
    from hf_cpu_amd.config import config_from_dict
    for cfg in (gh.SMALL, gh.CORES):
        c = config_from_dict(cfg)
        assert c.architecture == "Gitasun" and c.width == cfg["width"] and c.residual_mult == cfg["residual_mult"]
        for lc, raw in zip(c.layers, cfg["layers"]):
            assert lc.type == raw["type"] and (lc.mlp is None) == (raw["mlp"] is None)
            m = raw["mixer"]
            if lc.type == "latent_attention":
                assert (lc.mixer.heads, lc.mixer.dim, lc.mixer.rot_dim, lc.mixer.vdim, lc.mixer.kv_rank, lc.mixer.q_rank) == \
                    (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"])
                assert lc.mixer.rot.dims == m["rot"]["dims"] and lc.mixer.rot.base == m["rot"]["base"] and lc.mixer.scale == m["scale"]
                assert (lc.mixer.rot.scaling is None) == ("scaling" not in m["rot"])
            elif lc.type == "parallel":
                assert lc.mixer.left.kv_heads == m["left"]["kv_heads"] and lc.mixer.left.softcap == m["left"].get("softcap", 0.0)
                assert lc.mixer.right.tau == m["right"]["tau"] and lc.mixer.left_scale == m["left_scale"]
            if lc.mlp is not None and raw["mlp"]["kind"] == "moe":
                assert (lc.mlp.experts, lc.mlp.top, lc.mlp.ff) == (raw["mlp"]["router"]["experts"], raw["mlp"]["router"]["top"], raw["mlp"]["expert"]["ff"])
                assert lc.mlp.shared_ff == (raw["mlp"].get("shared") or {}).get("ff", 0)
        assert c.to_dict() == cfg


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="conv"), "conv"),
    (lambda c: c["layers"][2]["mixer"]["left"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3), "dims"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "choices"),
    (lambda c: c["layers"][2]["mlp"].update(kind="sparse"), "sparse"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][2]["mixer"]["right"].pop("tau"), "tau"),
])
def test_configuration_errors_name_the_key(change, word):
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.status import EngineError
    cfg = copy.deepcopy(gh.SMALL)
    change(cfg)
    with pytest.raises(EngineError) as e:
        config_from_dict(cfg)
    assert word in str(e.value.msg)


def test_plan_declares_the_tensors_of_a_checkpoint():
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.model import Model
    from hf_cpu_amd.parts.base import FixedState, PagedKV
    for cfg in (gh.SMALL, gh.CORES):
        model = Model.from_config(config_from_dict(cfg))
        declared = {s.name: s for s in model.param_specs()}
        made = gh.make_weights(cfg, 0)
        assert set(declared) == set(made)
        for name, s in declared.items():
            assert len(s.shape) == np.ndim(made[name]) and all(a == 0 or a == b for a, b in zip(s.shape, np.shape(made[name]))), name
        needs = model.cache_needs()
        kinds = []
        for lc in cfg["layers"]:
            kinds += {"latent_attention": [PagedKV], "hgrn2": [FixedState], "parallel": [PagedKV, FixedState]}[lc["type"]]
        assert [type(n) for n in needs] == kinds
        lat = [n for n, lc in zip(needs, cfg["layers"]) if lc["type"] == "latent_attention"]
    m = gh.CORES["layers"][0]["mixer"]
    first = Model.from_config(config_from_dict(gh.CORES)).cache_needs()[0]
    # one row a token: the rotated part and the latent as the key, the latent as the value, whatever the number of heads
    assert (first.k_width, first.v_width) == (m["rot_dim"] + m["kv_rank"], m["kv_rank"])
