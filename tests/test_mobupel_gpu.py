"""Mobupel in the engine against its plain implementation (tests/plain_mobupel.py): each mechanism alone at the
kernels, then whole models in every way of cutting the work."""
import math
import types

import numpy as np
import pytest
import torch

import helpers
import mobupel_helpers as mh
import plain_mobupel as pm
from test_kernels_gpu import FakeCache, FakeStep, dev, from_value_layout, ints, rounded, to_value_layout

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
# Largest |logit difference| from the float64 plain implementation, as a fraction of the request's largest |logit|.
# fp32: the rounding of fused multiply-adds and exponentials along a few hundred steps of two recurrences; a lost state,
# a tap too many, a head's weights on the wrong values or a gate left out shows as 1e-2 and more (measured: 1e-6 at most
# positions, 5.4e-5 at the worst, one of those where a head's read-out is small before it is divided by its root mean square).
# bf16: activations and cache rounded to 8 bits of mantissa at every part. The design divides the read-out of every head of
# its recurrences by the head's root mean square, and at a sequence's first tokens that read-out is one value vector times
# q . k, whose sign a rounding can turn where it is near zero; such places are off by tens of percent in any 16-bit
# implementation while their neighbours are within a percent or two. In bf16 the comparison is therefore one of the
# distribution (``compare_rounded``): the median within half the tolerance, at most one position in twelve beyond it and none
# beyond ten times it. (Measured: width 256: median 0.9e-2, 99 of 100 within 3e-2, worst 0.11; width 40: median 1.9e-2, 95 of
# 100 within 7.4e-2, worst 0.41.) What would differ between the dtypes' code paths (the matrix-core kernels) is held to its
# plain counterpart position by position in the tests of the mechanisms above.
TOL = {"float32": 1e-4, "bfloat16": 4e-2}
TOL_OF = {("small", "bfloat16"): 8e-2}


def compare_rounded(got, want, tol, what=""):
    errs = np.array([float(np.max(np.abs(row.astype(np.float64) - want[r][pos]))) / float(np.max(np.abs(want[r]))) for (r, pos), row in got.items()])
    assert np.median(errs) <= tol / 2, f"{what}: the median difference {np.median(errs):.3e} is beyond {tol / 2:.1e}"
    assert np.mean(errs > tol) <= 1.0 / 12, f"{what}: {int(np.sum(errs > tol))} of {len(errs)} positions differ by more than {tol:.1e}"
    assert errs.max() <= 10 * tol, f"{what}: a position differs by {errs.max():.3e}"
    return float(errs.max())


def compare_for(dtype, got, want, tol, what):
    return helpers.compare(got, want, tol, what) if dtype == "float32" else compare_rounded(got, want, tol, what)


def state_step(q_lens, slots):
    """What the kernels with per-request state read of a step: request ranges and state rows."""
    starts = np.concatenate([[0], np.cumsum(q_lens)])
    return types.SimpleNamespace(q_start=ints(starts), seq_slot=ints(slots), n_seqs=len(q_lens), max_q_len=int(max(q_lens)),
                                 n_tokens=int(starts[-1]))


def rel_err(got, want):
    return float(np.max(np.abs(np.asarray(got, np.float64) - want)) / max(1e-30, np.max(np.abs(want))))


# ---- mechanisms alone ----------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [6, 40, 77, 256, 1000])
def test_embedding_scaled_with_a_position_vector(ops32, dtype, width):
    rng = np.random.default_rng(width)
    V, T = 53, 19
    table = rounded(rng.standard_normal((V, width)), dtype)
    toks = rng.integers(0, V, T)
    positions = np.array([0, 1, 2, 3, 500, 4095, 17, 0, 1] + list(rng.integers(0, 3000, T - 9)))
    inv = 10000.0 ** (-2.0 * np.arange((width + 1) // 2) / width)
    out = torch.empty((T, width), dtype=torch.float32, device="cuda")
    ops32.embed(dev(table, dtype), ints(toks), out, scale=2.5, positions=ints(positions), inv_freq=dev(inv))
    want = table[toks] * 2.5 + pm.sinusoid(positions, width)
    # the angle is an fp32 product of a position up to 4,095 and a frequency: its rounding is what remains
    assert np.max(np.abs(out.cpu().numpy() - want)) <= 4096 * 2.0 ** -23
    ops32.embed(dev(table, dtype), ints(toks), out, scale=0.5)
    assert np.max(np.abs(out.cpu().numpy() - table[toks] * 0.5)) <= 1e-6


@pytest.mark.parametrize("width", [5, 40, 200, 1000, 4096])
def test_gated_norm_into_the_stream(ops32, width):
    """out (+)= scale * norm(y * sigmoid(gate + bias)) * w, the gate in either dtype and inside wider rows."""
    rng = np.random.default_rng(width)
    R, eps = 9, 1e-5
    y = (rng.standard_normal((R, width)) * rng.uniform(0.01, 30.0, (R, 1))).astype(np.float32)
    w, bias = (1.0 + 0.2 * rng.standard_normal(width)).astype(np.float32), rng.standard_normal(width).astype(np.float32)
    x0 = rng.standard_normal((R, width)).astype(np.float32)
    for gdt in DTYPES:
        wide = rounded(rng.standard_normal((R, width + 5)) * 2.0, gdt)
        gate = dev(wide, gdt)[:, 2:2 + width]
        for b in (None, bias):
            want = pm.rms_norm(y * pm.sigmoid(wide[:, 2:2 + width] + (0.0 if b is None else b)), w, eps)
            out = dev(x0)
            ops32.rmsnorm_add(dev(y), dev(w), eps, out, gate=gate, gate_bias=None if b is None else dev(b))
            assert np.max(np.abs(out.cpu().numpy() - (x0 + want))) <= 2e-5
            ops32.rmsnorm_add(dev(y), dev(w), eps, out, gate=gate, gate_bias=None if b is None else dev(b), scale=0.5, accumulate=False)
            assert np.max(np.abs(out.cpu().numpy() - 0.5 * want)) <= 2e-5
    out = dev(x0)
    ops32.rmsnorm_add(dev(y), dev(w), eps, out, scale=0.5)
    assert np.max(np.abs(out.cpu().numpy() - (x0 + 0.5 * pm.rms_norm(y.astype(np.float64), w, eps)))) <= 2e-5
    # a branch of zeros adds nothing (eps is inside the root)
    out = dev(x0)
    ops32.rmsnorm_add(torch.zeros((R, width), device="cuda"), dev(w), eps, out)
    assert np.array_equal(out.cpu().numpy(), x0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("F", [4, 24, 320, 1000, 8192])
def test_activation_of_normed_powers(ops32, dtype, F):
    rng = np.random.default_rng(F)
    z = (rng.standard_normal((7, F)) * rng.uniform(0.05, 8.0, (7, 1))).astype(np.float32)
    z[3] = 0.0
    coef = np.array([0.75, -0.5, 0.25, 0.125], np.float32)
    out = torch.empty((7, F), dtype=dtype, device="cuda")
    ops32.polynorm(dev(z), dev(coef), 1e-6, out)
    want = pm.poly_norm(z.astype(np.float64), coef, 1e-6)
    assert np.max(np.abs(out.float().cpu().numpy() - want) / (np.abs(want) + 1.0)) <= (1e-5 if dtype == torch.float32 else 1e-2)
    assert np.allclose(out.float().cpu().numpy()[3], 0.125)


@pytest.mark.parametrize("C,K", [(5, 2), (33, 4), (7, 1), (400, 3), (64, 8)])
def test_short_convolution_without_bias_or_activation(ops32, C, K):
    """Portions of every size, also shorter than the taps reach back; one tap needs no state."""
    rng = np.random.default_rng(C * K)
    lengths, slots = [70, 9], [1, 0]
    cuts = [[1, 1, 2, 1, 60, 3, 2], [2, 1, 1, 1, 2, 2]]
    seqs = [rng.standard_normal((n, C)).astype(np.float32) for n in lengths]
    taps = rng.standard_normal((C, K)).astype(np.float32)
    want = [pm.causal_conv(u.astype(np.float64), taps.astype(np.float64)) for u in seqs]
    state = torch.zeros((3, max(1, (K - 1) * C)), dtype=torch.float32, device="cuda")
    at, got = [0, 0], [np.zeros_like(u) for u in want]
    for turn in range(max(len(c) for c in cuts)):
        live = [s for s in range(2) if turn < len(cuts[s])]
        rows = np.concatenate([seqs[s][at[s]:at[s] + cuts[s][turn]] for s in live])
        out = torch.empty((rows.shape[0], C), dtype=torch.float32, device="cuda")
        ops32.causal_conv(dev(rows), dev(taps), None, state, state_step([cuts[s][turn] for s in live], [slots[s] for s in live]), out)
        o, r0 = out.cpu().numpy(), 0
        for s in live:
            n = cuts[s][turn]
            got[s][at[s]:at[s] + n] = o[r0:r0 + n]
            at[s], r0 = at[s] + n, r0 + n
    for s in range(2):
        assert np.max(np.abs(got[s] - want[s])) <= 2e-5, f"request {s}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,page", [(6, 3, 10, 6, 8), (4, 4, 8, 12, 4), (8, 2, 64, 64, 16), (4, 2, 128, 128, 16), (5, 1, 48, 20, 16)])
def test_queries_and_keys_normed_head_by_head_and_stored(ops32, ops16, dtype, H, G, D, Dv, page):
    """Every head of q and k over its own values with one weight for all heads; k and v land in the cache at the rows the
    step names, values transposed inside their page; rows in fp32 (after a convolution) and in the activations' dtype."""
    ops = ops32 if dtype == torch.float32 else ops16
    rng = np.random.default_rng(H * D + Dv)
    T, eps = 21, 1e-5
    QD, KD, VD = H * D, G * D, G * Dv
    qw, kw = (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32), (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)
    n_rows = 8 * page
    slot_map = rng.permutation(n_rows)[:T]
    for in_dtype in (torch.float32, dtype):
        rows = rounded(rng.standard_normal((T, QD + KD + VD)) * rng.uniform(0.1, 9.0, (T, 1)), in_dtype)
        cache = FakeCache(group=0, k=torch.zeros((n_rows, KD), dtype=dtype, device="cuda"), v=torch.zeros((n_rows, VD), dtype=dtype, device="cuda"),
                          page_tokens=page, window=0)
        q_out = torch.empty((T, QD), dtype=dtype, device="cuda")
        wide = torch.zeros((T, QD + KD + VD + 8), dtype=in_dtype, device="cuda")
        wide[:, :QD + KD + VD] = dev(rows, in_dtype)
        ops.head_norm_store(wide[:, :QD + KD + VD], H, G, D, Dv, dev(qw), dev(kw), eps, q_out, cache, ints(slot_map))
        want_q = pm.rms_norm(rows[:, :QD].reshape(T, H, D), qw, eps).reshape(T, QD)
        want_k = pm.rms_norm(rows[:, QD:QD + KD].reshape(T, G, D), kw, eps).reshape(T, KD)
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        assert np.max(np.abs(q_out.float().cpu().numpy() - want_q) / (np.abs(want_q) + 1.0)) <= tol
        assert np.max(np.abs(cache.k.float().cpu().numpy()[slot_map] - want_k) / (np.abs(want_k) + 1.0)) <= tol
        v_rows = from_value_layout(cache.v.float().cpu().numpy(), page)
        assert np.max(np.abs(v_rows[slot_map] - rows[:, QD + KD:]) / (np.abs(rows[:, QD + KD:]) + 1.0)) <= tol
        untouched = np.setdiff1d(np.arange(n_rows), slot_map)
        assert not cache.k.float().cpu().numpy()[untouched].any() and not v_rows[untouched].any()


def paged_kv(rng, lengths, G, D, Dv, page, dtype):
    """Keys and values of requests scattered over pages in a random order, the pages between them holding large values."""
    blocks = [-(-n // page) for n in lengths]
    n_pages = sum(blocks) + 3
    perm = rng.permutation(n_pages)
    table = np.zeros((len(lengths), max(blocks) + 2), np.int32)
    kc = np.full((n_pages * page, G * D), 1e4, np.float32)
    vc = np.full((n_pages * page, G * Dv), -1e4, np.float32)
    ks, vs, at = [], [], 0
    for s, n in enumerate(lengths):
        k, v = rng.standard_normal((n, G, D)).astype(np.float32), rng.standard_normal((n, G, Dv)).astype(np.float32)
        for b in range(blocks[s]):
            pg, at = perm[at], at + 1
            table[s, b] = pg
            rows = slice(b * page, min((b + 1) * page, n))
            cnt = rows.stop - rows.start
            kc[pg * page:pg * page + cnt] = k[rows].reshape(cnt, G * D)
            vc[pg * page:pg * page + cnt] = v[rows].reshape(cnt, G * Dv)
        ks.append(k)
        vs.append(v)
    return ks, vs, kc, vc, table


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,page", [(6, 3, 10, 6, 8), (4, 4, 8, 12, 4), (8, 2, 64, 64, 16), (4, 1, 32, 32, 16), (6, 2, 128, 128, 32),
                                           (8, 4, 96, 96, 16), (5, 5, 48, 48, 16), (3, 1, 64, 24, 16), (6, 3, 64, 64, 8), (32, 2, 32, 32, 4), (9, 3, 128, 128, 64),
                                           (16, 8, 64, 64, 16), (12, 6, 32, 32, 8), (32, 8, 128, 128, 16)])
def test_attention_weights_mixed_across_heads(ops32, ops16, dtype, H, G, D, Dv, page):
    """Portions of prompts and single tokens at the end of requests of many lengths, one of them long enough that a decoded
    token's keys are cut over several waves; in each request one query's head and one far key are scaled so that this key
    takes nearly all of that head's weight, which the mix then spreads over the heads; a gate inside wider rows."""
    ops = ops32 if dtype == torch.float32 else ops16
    rng = np.random.default_rng(H * 100 + D + page)
    lengths, q_lens = [1, 5, 64, 130, 203, 1500], [1, 3, 64, 1, 17, 1]
    ks, vs, kc, vc, table = paged_kv(rng, lengths, G, D, Dv, page, dtype)
    talk = (rng.standard_normal((H, H)) * 0.5 + np.eye(H)).astype(np.float32)
    scale = 1.3 / math.sqrt(D)
    qs, positions, slots, wants = [], [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q_full = rng.standard_normal((n, H, D)).astype(np.float32)
        if n > 100:                                 # key 3 of the last query's head 1 stands out among hundreds
            far, g = 3, 1 // (H // G)
            ks[s][far, g] *= 3.0
            q_full[n - 1, 1] = ks[s][far, g] * (12.0 / scale / float(ks[s][far, g] @ ks[s][far, g]))
            pg = table[s, far // page]
            kc[pg * page + far % page] = ks[s][far].reshape(-1)
            sc = scale * (ks[s][:, g].astype(np.float64) @ q_full[n - 1, 1].astype(np.float64))
            assert np.exp(sc[far] - sc.max()) / np.exp(sc - sc.max()).sum() > 0.5, "the far key was meant to stand out"
        full = pm.talking_attention(rounded(q_full, dtype), rounded(ks[s], dtype), rounded(vs[s], dtype), scale, talk.astype(np.float64))
        qs.append(q_full[n - ql:])
        wants.append(full[n - ql:])
        positions += list(range(n - ql, n))
        slots += [s] * ql
    cache = FakeCache(group=0, k=dev(kc, dtype), v=dev(to_value_layout(vc, page), dtype), page_tokens=page, window=0)
    q = np.concatenate(qs).reshape(-1, H * D)
    T = q.shape[0]
    gate_rows = rounded(rng.standard_normal((T, H * Dv + 16)) * 2.0, dtype)
    want = np.concatenate(wants).reshape(T, H * Dv)
    step = FakeStep(ints(positions), ints(slots), ints(table), None)
    tol = (3e-5 if dtype == torch.float32 else 0.02) * float(np.max(np.abs(want)))
    for plain_kernel in ([False] if dtype == torch.float32 else [False, True]):
        cross = torch.empty((T, G * H * Dv), dtype=dtype, device="cuda")
        ops.force_plain_attention = plain_kernel
        try:
            ops.paged_attention(dev(q, dtype), H, G, D, cache, step, 0, scale, cross, v_head_dim=Dv, cross_values=True)
        finally:
            ops.force_plain_attention = False
        out = torch.empty((T, H * Dv + 8), dtype=dtype, device="cuda")[:, :H * Dv]
        ops.talk_mix(cross, dev(talk), H, G, Dv, out)
        assert np.max(np.abs(out.float().cpu().numpy() - want)) <= tol, f"plain={plain_kernel}"
        ops.talk_mix(cross, dev(talk), H, G, Dv, out, gate=dev(gate_rows, dtype)[:, 16:])
        assert np.max(np.abs(out.float().cpu().numpy() - want * pm.sigmoid(gate_rows[:, 16:]))) <= tol, f"plain={plain_kernel}"
    # single tokens alone (a decode step): in bf16, where the sizes allow, one pass over the cache for all groups' values
    ends = np.cumsum(q_lens) - 1
    step1 = FakeStep(ints([n - 1 for n in lengths]), ints(list(range(len(lengths)))), ints(table), None)
    cross = torch.empty((len(lengths), G * H * Dv), dtype=dtype, device="cuda")
    ops.paged_attention(dev(q[ends], dtype), H, G, D, cache, step1, 0, scale, cross, v_head_dim=Dv, cross_values=True)
    out = torch.empty((len(lengths), H * Dv), dtype=dtype, device="cuda")
    ops.talk_mix(cross, dev(talk), H, G, Dv, out)
    assert np.max(np.abs(out.float().cpu().numpy() - want[ends])) <= tol, "single tokens"


def scan_in_portions(q, cuts, slots, n_state, call):
    """Runs ``call(step, live requests, their slices, state)`` portion by portion; returns each request's rows."""
    T = [len(x) for x in q]
    state = torch.zeros((max(slots) + 2, n_state), dtype=torch.float32, device="cuda")
    at, got = [0] * len(q), [None] * len(q)
    for turn in range(max(len(c) for c in cuts)):
        live = [s for s in range(len(q)) if turn < len(cuts[s])]
        take = {s: slice(at[s], at[s] + cuts[s][turn]) for s in live}
        out = call(state_step([cuts[s][turn] for s in live], [slots[s] for s in live]), live, take, state)
        r0 = 0
        for s in live:
            n = cuts[s][turn]
            got[s] = out[r0:r0 + n] if got[s] is None else np.concatenate([got[s], out[r0:r0 + n]])
            at[s], r0 = at[s] + n, r0 + n
    assert at == T
    return got, state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,P,cap", [(3, 6, 10, 5.0), (1, 12, 4, 1.0), (4, 64, 64, 15.0), (2, 128, 64, 10.0), (8, 32, 32, 20.0), (2, 32, 40, 12.0),
                                       (2, 200, 8, 3.0), (1, 16, 255, 50.0)])
def test_matrix_memory_in_portions(ops32, dtype, H, D, P, cap):
    """Capped exponential input gates and sigmoid forget gates under a running maximum that starts at 0, the normaliser
    beside the state: three requests in portions down to one token against the recurrence over the whole sequences; a run
    of input gates far below 0 at the start (the maximum stays 0), one far above later (everything before shrinks); then a
    request in a state row that another has used (cleared, as at admission)."""
    rng = np.random.default_rng(H * D + P)
    lengths, cuts, slots = [300, 5, 33], [[1, 2, 17, 1, 200, 79], [2, 3], [16, 1, 16]], [1, 3, 0]
    q = [rounded(rng.standard_normal((n, H, D)), dtype) for n in lengths]
    k = [rounded(rng.standard_normal((n, H, D)) * 0.7, dtype) for n in lengths]
    v = [rounded(rng.standard_normal((n, H, P)), dtype) for n in lengths]
    gi = [(rng.standard_normal((n, H)) * 2.0).astype(np.float32) for n in lengths]
    gf = [(rng.standard_normal((n, H)) * 2.0 + 2.0).astype(np.float32) for n in lengths]
    gi[0][:4] = -6.0 * cap
    gi[0][40, 0], gf[0][41, 0] = 8.0 * cap, -9.0 * cap
    ib, fb = rng.standard_normal(H).astype(np.float32), rng.standard_normal(H).astype(np.float32)
    qs = D ** -0.5

    def whole(s):
        li = pm.soft_cap(gi[s].astype(np.float64) + ib, cap)
        lf = pm.log_sigmoid(pm.soft_cap(gf[s].astype(np.float64) + fb, cap))
        return pm.mlstm_scan(q[s] * qs, k[s], v[s], li, lf).reshape(lengths[s], -1)
    want = [whole(s) for s in range(3)]
    QD = H * D

    def call(step, live, take, state):
        rows = lambda parts, width: np.concatenate([parts[s][take[s]].reshape(-1, width) for s in live])
        qkv = dev(np.concatenate([rows(q, QD), rows(k, QD), rows(v, H * P)], axis=1), dtype)
        gates = dev(np.concatenate([rows(gi, H), rows(gf, H)], axis=1))
        T = step.n_tokens
        y = torch.empty((T, H * P), dtype=torch.float32, device="cuda")
        denom = torch.empty((T, H), dtype=torch.float32, device="cuda")
        ops32.linear_scan(qkv[:, :QD], qkv[:, QD:2 * QD], qkv[:, 2 * QD:], H, D, H, P, state, step, y,
                          exp_gates=(gates[:, :H], gates[:, H:], dev(ib), dev(fb), cap), q_scale=qs, denom=denom)
        return (y.view(T, H, P) * denom.view(T, H, 1)).reshape(T, H * P).cpu().numpy()
    n_state = ops32.scan_state_floats(H, D, P, normalizer=True)
    assert n_state >= H * (D * (P + 1) + 1)
    got, state = scan_in_portions(q, cuts, slots, n_state + 3, call)
    for s in range(3):
        assert rel_err(got[s], want[s]) <= 3e-5, f"request {s}"
    state[0].zero_()
    again = call(state_step([lengths[1]], [0]), [1], {1: slice(0, lengths[1])}, state)
    assert rel_err(again, want[1]) <= 3e-5


@pytest.mark.parametrize("H,G,N,P", [(4, 2, 7, 5), (3, 3, 12, 4), (6, 1, 4, 9), (4, 2, 64, 64), (2, 2, 128, 32), (8, 4, 32, 64), (4, 4, 64, 16),
                                     (2, 1, 200, 8), (1, 1, 16, 255)])
def test_gated_delta_rule_in_portions(ops32, H, G, N, P):
    """Unit queries and keys, a decay per key channel through softplus and two exponentials, a write strength through the
    logistic function: three requests in portions down to one token against the recurrence over the whole sequences;
    softplus far from zero on both sides; a key repeated so that the correction towards the new value shows."""
    rng = np.random.default_rng(H * N + P)
    lengths, cuts, slots = [260, 5, 33], [[1, 2, 17, 1, 160, 79], [2, 3], [16, 1, 16]], [1, 3, 0]
    q = [rng.standard_normal((n, G, N)).astype(np.float32) for n in lengths]
    k = [rng.standard_normal((n, G, N)).astype(np.float32) for n in lengths]
    v = [rng.standard_normal((n, H, P)).astype(np.float32) for n in lengths]
    k[0][100:110] = k[0][100]                                    # ten writes at one key
    q[0][109] = k[0][100]
    a = [(rng.standard_normal((n, H * N)) * 1.5).astype(np.float32) for n in lengths]
    a[0][3, :N], a[0][4, :N] = 60.0, -60.0
    b = [(rng.standard_normal((n, H)) * 2.0).astype(np.float32) for n in lengths]
    dt_bias, a_log = (rng.standard_normal(H * N) - 1.0).astype(np.float32), (rng.standard_normal(H) * 0.7 - 0.5).astype(np.float32)
    qs, eps = N ** -0.5, 1e-6

    def whole(s):
        f64 = lambda x: x.astype(np.float64)
        decay = np.exp(-np.exp(f64(a_log))[None, :, None] * pm.softplus(f64(a[s]) + dt_bias).reshape(-1, H, N))
        return pm.delta_scan(pm.unit(f64(q[s]), eps) * qs, pm.unit(f64(k[s]), eps), f64(v[s]), pm.sigmoid(f64(b[s])), decay).reshape(lengths[s], -1)
    want = [whole(s) for s in range(3)]

    def call(step, live, take, state):
        rows = lambda parts, width: np.concatenate([parts[s][take[s]].reshape(-1, width) for s in live])
        qkv = dev(np.concatenate([rows(q, G * N), rows(k, G * N), rows(v, H * P)], axis=1))      # one matrix, as the mixer holds them
        y = torch.empty((step.n_tokens, H * P), dtype=torch.float32, device="cuda")
        ops32.delta_scan(qkv[:, :G * N], qkv[:, G * N:2 * G * N], qkv[:, 2 * G * N:], G, N, H, P, dev(rows(a, H * N)), dev(dt_bias), dev(a_log),
                         dev(rows(b, H)), state, step, y, q_scale=qs, unit_eps=eps)
        return y.cpu().numpy()
    got, state = scan_in_portions(q, cuts, slots, ops32.scan_state_floats(H, N, P) + 5, call)
    for s in range(3):
        assert rel_err(got[s], want[s]) <= 3e-5, f"request {s}"
    state[0].zero_()
    again = call(state_step([lengths[1]], [0]), [1], {1: slice(0, lengths[1])}, state)
    assert rel_err(again, want[1]) <= 3e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_of_heads_with_a_factor_a_head(ops32, dtype):
    """The read-out of the matrix memory: every head's row times its denominator, divided by its root mean square, times the
    weight, times the logistic function of the gate."""
    rng = np.random.default_rng(11)
    T, H, P = 9, 3, 10
    y, d = rng.standard_normal((T, H * P)).astype(np.float32), rng.uniform(0.01, 5.0, (T, H)).astype(np.float32)
    w, gate = (1.0 + 0.2 * rng.standard_normal(H * P)).astype(np.float32), rounded(rng.standard_normal((T, H * P)), dtype)
    out = torch.empty((T, H * P), dtype=dtype, device="cuda")
    ops32.group_rmsnorm(dev(y), dev(w), 1e-5, H, out, gate=dev(gate, dtype), gate_kind="sigmoid_after", row_scale=dev(d))
    o = (y.reshape(T, H, P).astype(np.float64) * d[:, :, None])
    want = pm.rms_div(o, 1e-5).reshape(T, H * P) * w * pm.sigmoid(gate)
    assert np.max(np.abs(out.float().cpu().numpy() - want) / (np.abs(want) + 1.0)) <= (1e-5 if dtype == torch.float32 else 1e-2)


# ---- whole models ---------------------------------------------------------------------------------------------------

LENGTHS = {"small": [1, 2, 3, 23, 24, 57, 130], "cores": [3, 48, 49, 97, 161, 230]}


@pytest.fixture(scope="module", params=["small", "cores"])
def tiny(request, tmp_path_factory):
    name = request.param
    cfg = mh.CONFIGS[name]
    d = mh.make_model_dir(str(tmp_path_factory.mktemp("mobupel_" + name)), cfg, seed=len(name), stored=mh.STORED[name])
    reqs = mh.random_requests(cfg, LENGTHS[name], seed=7)
    return name, cfg, d, reqs, mh.plain_logits(d, reqs)


def engine_for(model_dir, dtype, name, max_tokens, max_seqs=4, graphs=True):
    import hf_cpu_amd
    return hf_cpu_amd.load_engine(model_dir, dtype=dtype, page_tokens=mh.PAGE[name], max_tokens=max_tokens, max_seqs=max_seqs, graphs=graphs)


def run_against_plain(name, d, reqs, want, dtype, steps, what, graphs=True):
    engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps), graphs=graphs)
    got = helpers.run_trace_in_engine(engine, steps)
    worst = compare_for(dtype, got, want, TOL_OF.get((name, dtype), TOL[dtype]), what)
    engine.manager.check()
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)
    return engine, got, worst


def test_the_stream_after_every_layer(gpu, tiny):
    """Layer by layer in fp32: the stream after each layer of a prompt against the plain implementation's."""
    from hf_cpu_amd.parts.block import SandwichBlock
    name, cfg, d, reqs, _ = tiny
    toks = reqs["r3"]
    pcfg, w = pm.read_model(d)
    want = []
    pm.forward(pcfg, w, toks, layers_out=want)
    engine = engine_for(d, "float32", name, 256, graphs=False)
    caught, orig = [], SandwichBlock.forward

    def fwd(self, ops, step, x, parts, caches, write_cache=True):
        orig(self, ops, step, x, parts, caches, write_cache)
        ops.settle()
        caught.append(x.clone())
    SandwichBlock.forward = fwd
    try:
        engine.step([("a", toks, [len(toks) - 1])])
    finally:
        SandwichBlock.forward = orig
    assert len(caught) == len(want)
    for l, (x, ref) in enumerate(zip(caught, want)):
        assert rel_err(x.cpu().numpy(), ref) <= 2e-5, f"{name}: layer {l} ({cfg['layers'][l]['type']})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cutting", ["whole", "tail", "portions", "mixed"])
def test_cuttings(gpu, tiny, dtype, cutting):
    """Whole prompts; most of a prompt and then token by token; portions of changing size down to two tokens; up to
    four requests live, portions beside single tokens, pages and state rows used again."""
    name, cfg, d, reqs, want = tiny
    steps = {"whole": helpers.trace_whole, "tail": lambda r: helpers.trace_tail(r, tail=90),
             "portions": helpers.trace_portions, "mixed": lambda r: helpers.trace_mixed(r, seed=3)}[cutting](reqs)
    engine, got, worst = run_against_plain(name, d, reqs, want, dtype, steps, f"{name} {dtype} {cutting}")
    assert len(got) == sum(len(t) for t in reqs.values())
    print(f"{name} {dtype} {cutting}: worst |diff| {worst:.3e}")
    if cutting == "mixed":
        assert any(p.reused > 0 for p in engine.manager.pools), "the trace was meant to use pages again"


def test_cuttings_agree_with_each_other(gpu, tiny):
    """In fp32 the cuttings agree among themselves far more closely than rounding in bf16 would allow: the same values
    are computed, only in other launches; decoding replays captured graphs."""
    name, cfg, d, reqs, _ = tiny
    results = []
    for make in (helpers.trace_whole, helpers.trace_portions, lambda r: helpers.trace_tail(r, tail=60),
                 lambda r: helpers.trace_mixed(r, seed=5), lambda r: helpers.trace_portions(r, sizes=(2, 2, 3, 2, 64, 2, 7))):
        steps = make(reqs)
        engine = engine_for(d, "float32", name, helpers.max_live_tokens(steps))
        results.append(helpers.run_trace_in_engine(engine, steps))
    for other in results[1:]:
        for key, row in results[0].items():
            err = float(np.max(np.abs(row - other[key])))
            assert err <= 5e-5 * max(1.0, float(np.max(np.abs(row)))), f"{name}: {key}: cuttings differ by {err:.3e}"


def test_a_batch_of_unequal_requests_against_each_alone(gpu, tiny):
    name, cfg, d, reqs, want = tiny
    engine = engine_for(d, "float32", name, 64 * len(reqs) + sum(len(t) for t in reqs.values()), max_seqs=len(reqs))
    together = engine.step([(r, toks, list(range(len(toks)))) for r, toks in reqs.items()]).cpu().numpy()
    at = 0
    for r, toks in reqs.items():
        engine.release(r)
        alone = engine.step([(r + "'", toks, list(range(len(toks))))]).cpu().numpy()
        engine.release(r + "'")
        assert np.max(np.abs(alone - together[at:at + len(toks)])) <= 5e-5 * np.max(np.abs(want[r]))
        assert np.max(np.abs(alone - want[r])) <= TOL["float32"] * np.max(np.abs(want[r]))
        at += len(toks)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_small_pool(gpu, tiny, dtype):
    """Three requests decoded token by token together from their second token on, in a pool that holds them and no
    more, then three more in the pages and state rows that they gave back: what the first left there must be gone."""
    name, cfg, d, reqs, want = tiny
    long = {r: t for r, t in reqs.items() if len(t) >= 57}
    names = list(long)[:3]
    order = [names, names[::-1]]                    # the second turn's requests land in other state rows than the first's
    steps = []
    for turn in range(2):
        ids = {r: f"{r}/{turn}" for r in names}
        steps.append(helpers._step(len(steps), [(ids[r], long[r][:2], [0, 1]) for r in order[turn]]))
        for i in range(2, max(len(long[r]) for r in names)):
            live = [r for r in order[turn] if i < len(long[r])]
            steps.append(helpers._step(len(steps), [(ids[r], long[r][i:i + 1], [0]) for r in live],
                                       [ids[r] for r in live if i == len(long[r]) - 1]))
    reqs2 = {f"{r}/{turn}": long[r] for r in names for turn in range(2)}
    want2 = {f"{r}/{turn}": want[r] for r in names for turn in range(2)}
    engine, got, _ = run_against_plain(name, d, reqs2, want2, dtype, steps, f"{name} {dtype} long decoding")
    assert all(p.reused > 0 for p in engine.manager.pools)
    assert engine.graph_replays > 0, "decode steps were meant to replay captured graphs"


def test_trace_replay_program(gpu, tiny, tmp_path):
    """bin/trace_run as a user calls it (pages of 16, four state rows, a pool for the live requests only): a mixed trace
    against the plain implementation in both dtypes."""
    import json
    import os
    import subprocess
    import sys
    name, cfg, d, reqs, want = tiny
    steps = helpers.trace_mixed(reqs, seed=21)
    places = helpers.wanted_places(steps)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out),
                            "--max-tokens", str(helpers.max_live_tokens(steps))],
                           input="".join(json.dumps(st) + "\n" for st in steps), text=True, capture_output=True, timeout=300)
        assert r.returncode == 0, r.stderr
        assert [w for w in r.stdout.split() if w != "done"] == [str(st["step"]) for st in steps]
        got = {}
        for st in steps:
            if st["step"] in places:
                rows = np.fromfile(out / f"{st['step']}.f32", dtype="<f4").reshape(len(places[st["step"]]), -1)
                got.update(zip(places[st["step"]], rows))
        assert len(got) == sum(len(t) for t in reqs.values())
        compare_for(dtype, got, want, TOL_OF.get((name, dtype), TOL[dtype]), "trace_run " + dtype)


def test_greedy_generation_through_the_session(gpu, tiny):
    """Greedy continuation of three prompts through Session.generate (the scheduler, the sampler, graphs): every token
    is the plain implementation's best, or within rounding of it."""
    import hf_cpu_amd.session as S
    name, cfg, d, reqs, _ = tiny
    prompts = [reqs["r3"], reqs["r4"], reqs["r5"]]
    pcfg, w = pm.read_model(d)
    s = S.Session(d, dtype="float32", ctx_max=256, batch=16, page_size=mh.PAGE[name], max_seqs=4)
    gens = s.generate(prompts, temp=0.0, max_tokens=20)
    for g, p in zip(gens, prompts):
        assert len(g.tokens) == 20
        toks = list(p)
        for i, t in enumerate(g.tokens):
            row = pm.forward(pcfg, w, toks)[-1]
            assert row[int(np.argmax(row))] - row[t] <= 1e-4 * max(1.0, float(np.max(np.abs(row)))), \
                f"token {i} = {t}, plain picks {int(np.argmax(row))}"
            toks.append(t)


def far_key_model():
    """One side-by-side layer whose attention is made to look far back. The stream's last entry is the cosine of a tiny
    angle, always near 1 (the table's last two columns are zero), and the first head's queries are a fixed vector u times
    that entry, so after their norm all of them are u's direction. Token 1 alone has a large entry in the column before,
    which its key projection turns into a multiple of u: every query of the first head gives nearly all its weight to
    token 1's key, however far back, and the mix of heads hands that weight to the second head too. The delta rule's
    side is silenced."""
    E, D = 64, 32
    cfg = mh.config(50, E, [mh.layer(mh.parallel(mh.left(2, 1, D, D, 1, scale=1.0), mh.right(1, 1, 32, 32, 1)), None)], embedding_scale=1.0)
    w = mh.make_weights(cfg, seed=1)
    rng = np.random.default_rng(5)
    u = helpers.bf16_round(rng.standard_normal(D))
    p = "l0.mix.left."
    for n in "qkv":
        w[p + n + ".conv"][:] = 1.0
    w[p + "q.norm"][:], w[p + "k.norm"][:] = 1.0, 1.0
    w["embed"][:, E - 2:] = 0.0
    w["embed"][1, E - 2] = 30.0
    w["l0.norm1"][:] = 1.0
    w[p + "q"][:D] = 0.0
    w[p + "q"][:D, E - 1] = u
    w[p + "k"][:, E - 2] = 2.0 * u
    w["l0.mix.right.o"] = np.zeros_like(w["l0.mix.right.o"])
    return cfg, w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_far_back_among_hundreds(gpu, tmp_path, dtype):
    """A prompt of 900 tokens in two portions and 20 decoded tokens: the marked token stands at position 2, at the last
    place of a page, or nowhere; the plain logits of the late tokens differ widely between these, and the engine's are the
    plain ones in each."""
    import hf_cpu_amd
    cfg, w = far_key_model()
    d = mh.make_model_dir(str(tmp_path / "m"), cfg, seed=0, weights=w, stored="BF16")
    rng = np.random.default_rng(9)
    base = [int(t) for t in rng.integers(2, cfg["vocab"], 920)]
    reqs = {"none": base, "early": base[:2] + [1] + base[3:], "edge": base[:15] + [1] + base[16:]}
    want = mh.plain_logits(d, reqs)
    late = slice(600, 920)
    for r in ("early", "edge"):
        assert np.max(np.abs(want[r][late] - want["none"][late])) >= 0.1 * np.max(np.abs(want["none"])), "the plain logits do not show the far key"
    steps = []
    for r, t in reqs.items():
        steps.append(helpers._step(len(steps), [(r, t[:391], [2, 15, 390])]))
        steps.append(helpers._step(len(steps), [(r, t[391:900], list(range(300, 509, 16)))]))
        for i in range(900, 920):
            steps.append(helpers._step(len(steps), [(r, t[i:i + 1], [0])], [r] if i == 919 else []))
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=helpers.max_live_tokens(steps), max_seqs=1)
    got = helpers.run_trace_in_engine(engine, steps)
    compare_for(dtype, got, want, TOL[dtype], f"far key {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_decoded_token_by_token(gpu, tmp_path, dtype):
    """Two requests of 700 and 1,300 tokens: the prompt in two portions (the second begins in the middle of a page),
    then 45 tokens decoded together; attention cuts the keys of a decoded token over many waves, the states have been
    carried over a thousand steps."""
    import hf_cpu_amd
    cfg = mh.config(300, 128, [
        mh.layer(mh.parallel(mh.left(4, 1, 64, 64, 4), mh.right(2, 1, 64, 64, 4)), 128),
        mh.layer(mh.mlstm(2, 64, 64, 15.0), None),
        mh.layer(mh.parallel(mh.left(4, 2, 32, 32, 2), mh.right(2, 2, 32, 64, 3)), None),
        mh.layer(mh.mlstm(2, 32, 64, 15.0), 96)])
    d = mh.make_model_dir(str(tmp_path / "m"), cfg, seed=4, stored="BF16")
    reqs = mh.random_requests(cfg, [700, 1300], seed=2)
    want = mh.plain_logits(d, reqs)
    steps = []
    heads = {r: len(t) - 45 for r, t in reqs.items()}
    for r, t in reqs.items():
        steps.append(helpers._step(len(steps), [(r, t[:heads[r] - 201], [heads[r] - 202])]))
        steps.append(helpers._step(len(steps), [(r, t[heads[r] - 201:heads[r]], [0, 200])]))
    for i in range(45):
        steps.append(helpers._step(len(steps), [(r, t[heads[r] + i:heads[r] + i + 1], [0]) for r, t in reqs.items()],
                                   list(reqs) if i == 44 else []))
    engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=helpers.max_live_tokens(steps), max_seqs=2)
    got = helpers.run_trace_in_engine(engine, steps)
    assert len(got) == 2 * 48
    # (fp32: the rounding of two recurrences carried over 1,300 steps, measured 8e-5)
    compare_for(dtype, got, want, 2e-4 if dtype == "float32" else TOL[dtype], f"long prompts {dtype}")
    engine.manager.check()


def test_random_weights_and_other_orders_of_layers(gpu, tmp_path):
    """``write_random_model`` makes a folder for this design too (the low-rank projections' inner sizes from the
    configuration), and the engine reads it back: a model of one matrix memory, one of one side-by-side layer with a single
    head everywhere, and one with widths that are no multiple of 8."""
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    one = mh.config(90, 64, [mh.layer(mh.mlstm(1, 32, 32, 15.0), 16)])
    two = mh.config(90, 64, [mh.layer(mh.parallel(mh.left(1, 1, 32, 32, 2), dict(mh.right(1, 1, 32, 32, 2), decay_rank=4, gate_rank=6)), None)])
    odd = mh.config(77, 100, eps=1e-3, layers=[
        mh.layer(mh.parallel(mh.left(3, 1, 20, 28, 3), dict(mh.right(4, 2, 5, 3, 3), decay_rank=3, gate_rank=2)), 12),
        mh.layer(mh.mlstm(5, 4, 3, 2.0), None),
        mh.layer(mh.mlstm(2, 9, 7, 15.0), 20)])
    for k, c in enumerate((one, two, odd)):
        d = str(tmp_path / f"m{k}")
        hf_cpu_amd.write_random_model(d, config_from_dict(c), seed=3, dtype="bfloat16")
        pcfg, w = pm.read_model(d)
        toks = [int(t) for t in np.random.default_rng(0).integers(0, c["vocab"], 45)]
        want = pm.forward(pcfg, w, toks)
        for dtype in ("float32", "bfloat16"):
            engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=4, max_tokens=64, max_seqs=1)
            got = engine.step([("a", toks[:31], list(range(31)))]).cpu().numpy()
            rows = {("a", i): row for i, row in enumerate(got)}
            for i in range(31, 45):
                rows[("a", i)] = engine.step([("a", toks[i:i + 1], [0])]).cpu().numpy()[0]
            compare_for(dtype, rows, {"a": want}, TOL[dtype] if dtype == "float32" else 8e-2, f"random weights {k} {dtype}")


@pytest.mark.parametrize("seed", range(6))
def test_configurations_drawn_at_random(gpu, tmp_path, seed):
    """Layers of either kind in any order with sizes drawn at random (even seeds: sizes for the matrix cores): a prompt, a
    portion that starts in the middle of a page, then single tokens, in fp32 and in bf16."""
    import hf_cpu_amd
    rng = np.random.default_rng(100 + seed)
    cfg = mh.random_config(rng, big=seed % 2 == 0)
    d = mh.make_model_dir(str(tmp_path / "m"), cfg, seed=seed, stored="BF16" if seed % 2 == 0 else "F32")
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 110)]
    pcfg, w = pm.read_model(d)
    want = pm.forward(pcfg, w, toks)
    steps = [helpers._step(0, [("a", toks[:55], range(55))]), helpers._step(1, [("a", toks[55:88], range(33))])]
    steps += [helpers._step(2 + i, [("a", toks[88 + i:89 + i], [0])], ["a"] if i == 21 else []) for i in range(22)]
    for dtype in ("float32", "bfloat16"):
        engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=128, max_seqs=2, graphs=dtype == "float32")
        got = helpers.run_trace_in_engine(engine, steps)
        compare_for(dtype, got, {"a": want}, TOL[dtype] if dtype == "float32" else 8e-2, f"random configuration {seed} {dtype}: {cfg}")
