"""Gitasun in the engine against its plain implementation (tests/plain_gitasun.py): each mechanism alone at the
kernels, then whole models in every way of cutting the work."""
import math
import types

import numpy as np
import pytest
import torch

import helpers
import gitasun_helpers as gh
import plain_gitasun as pg
from test_kernels_gpu import FakeCache, FakeStep, dev, ints, rounded, to_value_layout

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
# Largest |logit difference| from the float64 plain implementation, as a fraction of the request's largest |logit|.
# fp32: the rounding of fused multiply-adds and exponentials along a few hundred steps of the recurrences; a lost state, a
# head's weights on the wrong values, a gate, a bias or a factor left out shows as 1e-2 and more.
# bf16: activations and cache rounded to 8 bits of mantissa at every part; the recurrences' read-outs are divided by their
# root mean square head by head, and where a read-out is small a rounding weighs more: the comparison is one of the
# distribution (``compare_rounded``): the median within half the tolerance, at most one position in twelve beyond it and none
# beyond ten times it.
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

@pytest.mark.parametrize("width", [5, 40, 200, 1000])
def test_branch_into_the_stream_with_a_factor_and_a_vector(ops32, width):
    rng = np.random.default_rng(width)
    R = 7
    y, x0 = rng.standard_normal((R, width)).astype(np.float32), rng.standard_normal((R, width)).astype(np.float32)
    col = rng.uniform(0.2, 1.5, width).astype(np.float32)
    wide = dev(np.zeros((R, width + 3), np.float32))
    wide[:, 1:1 + width] = dev(y)
    out = dev(x0)
    ops32.scale_add(wide[:, 1:1 + width], out, scale=0.7, columns=dev(col))
    assert np.max(np.abs(out.cpu().numpy() - (x0 + 0.7 * col * y.astype(np.float64)))) <= 1e-6
    ops32.scale_add(dev(y), out, scale=-1.25, accumulate=False)
    assert np.max(np.abs(out.cpu().numpy() - (-1.25 * y))) <= 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["sigmoid", "silu"])
def test_gate_on_the_heads(ops32, dtype, kind):
    rng = np.random.default_rng(3)
    x, g = rounded(rng.standard_normal((9, 44)), dtype), rounded(rng.standard_normal((9, 50)) * 3.0, dtype)
    xd, gd = dev(x, dtype), dev(g, dtype)[:, 3:47]
    act = pg.sigmoid if kind == "sigmoid" else pg.silu
    want = x * act(g[:, 3:47])
    ops32.gate_mul(xd, gd, xd, kind)                       # in place, the gate inside wider rows
    assert np.max(np.abs(xd.float().cpu().numpy() - want) / (np.abs(want) + 1.0)) <= (1e-6 if dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_of_heads_with_a_silu_gate_after(ops32, dtype):
    rng = np.random.default_rng(11)
    T, H, P = 9, 3, 10
    y = rng.standard_normal((T, H * P)).astype(np.float32)
    w, gate = (1.0 + 0.2 * rng.standard_normal(P)).astype(np.float32), rounded(rng.standard_normal((T, H * P)) * 2.0, dtype)
    out = torch.empty((T, H * P), dtype=dtype, device="cuda")
    ops32.group_rmsnorm(dev(y), dev(np.tile(w, H)), 1e-5, H, out, gate=dev(gate, dtype), gate_kind="silu_after")
    want = pg.rms_norm(y.reshape(T, H, P).astype(np.float64), w, 1e-5).reshape(T, H * P) * pg.silu(gate)
    assert np.max(np.abs(out.float().cpu().numpy() - want) / (np.abs(want) + 1.0)) <= (1e-5 if dtype == torch.float32 else 1e-2)


def test_rescaled_rotary_table(gpu, ops32):
    from hf_cpu_amd.parts.position import Rotary
    for dims, base, sc in ((40, 30000.0, (6.0, 1.0, 3.0, 256)), (6, 500.0, (4.0, 1.0, 3.0, 64)), (32, 10000.0, None), (64, 1e6, (32.0, 1.0, 4.0, 8192))):
        part = Rotary(head_dim=dims + 4, rot_dim=dims, theta=base, scaling=None if sc is None else dict(zip(("factor", "low", "high", "original"), sc)))
        part.bind({}, ops32)
        want = pg.rotary_frequencies(dims, base, None if sc is None else dict(zip(("factor", "low", "high", "original"), sc)))
        assert np.max(np.abs(part.inv_freq.cpu().numpy() / want - 1.0)) <= 2.0 ** -23


def scan_in_portions(lengths, cuts, slots, n_state, call):
    """Runs ``call(step, live requests, their slices, state)`` portion by portion; returns each request's rows."""
    state = torch.zeros((max(slots) + 2, n_state), dtype=torch.float32, device="cuda")
    at, got = [0] * len(lengths), [None] * len(lengths)
    for turn in range(max(len(c) for c in cuts)):
        live = [s for s in range(len(lengths)) if turn < len(cuts[s])]
        take = {s: slice(at[s], at[s] + cuts[s][turn]) for s in live}
        out = call(state_step([cuts[s][turn] for s in live], [slots[s] for s in live]), live, take, state)
        r0 = 0
        for s in live:
            n = cuts[s][turn]
            got[s] = out[r0:r0 + n] if got[s] is None else np.concatenate([got[s], out[r0:r0 + n]])
            at[s], r0 = at[s] + n, r0 + n
    assert at == list(lengths)
    return got, state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("form", ["forget", "tau"])
@pytest.mark.parametrize("H,D,P", [(3, 5, 7), (1, 20, 4), (4, 64, 64), (2, 128, 32), (2, 32, 40), (2, 200, 8), (1, 16, 255), (4, 48, 32)])
def test_recurrence_with_a_decay_per_key_channel_in_portions(ops32, dtype, form, H, D, P):
    """Three requests in portions down to one token against the recurrence over the whole sequences, for the forget gate
    that also writes (a lower bound per channel, queries through silu, no keys) and for decays that are a root of a sigmoid
    (keys read, queries scaled); gates far on either side (a channel that keeps everything, one that keeps nothing); then a
    request in a state row that another has used (cleared, as at admission)."""
    rng = np.random.default_rng(H * D + P)
    lengths, cuts, slots = [300, 5, 33], [[1, 2, 17, 1, 200, 79], [2, 3], [16, 1, 16]], [1, 3, 0]
    q = [rounded(rng.standard_normal((n, H, D)), dtype) for n in lengths]
    k = [rounded(rng.standard_normal((n, H, D)) * 0.7, dtype) for n in lengths]
    v = [rounded(rng.standard_normal((n, H, P)), dtype) for n in lengths]
    gdt = dtype if form == "forget" else torch.float32        # the forget gate's input rides in the mixer's one projection
    z = [rounded(rng.standard_normal((n, H * D)) * 2.0 + 1.0, gdt) for n in lengths]
    z[0][3, :D], z[0][4, :D] = 60.0, -60.0
    bias = (rng.standard_normal(H * D) * 0.5).astype(np.float32)
    lower = rng.uniform(0.0, 0.9, H * D).astype(np.float32)
    lower[0] = 0.0
    tau, qs = 16.0 if D % 2 else 3.0, D ** -0.5

    def whole(s):
        zz = (z[s] + bias).reshape(-1, H, D)
        if form == "forget":
            f = lower.reshape(H, D) + (1.0 - lower.reshape(H, D).astype(np.float64)) * pg.sigmoid(zz)
            return pg.channel_decay_recurrence(pg.silu(q[s]), 1.0 - f, v[s], f).reshape(lengths[s], -1)
        return pg.channel_decay_recurrence(q[s] * qs, k[s], v[s], pg.sigmoid(zz) ** (1.0 / tau)).reshape(lengths[s], -1)
    want = [whole(s) for s in range(3)]

    def call(step, live, take, state):
        rows = lambda parts, width: np.concatenate([parts[s][take[s]].reshape(-1, width) for s in live])
        qkv = dev(np.concatenate([rows(q, H * D), rows(k, H * D), rows(v, H * P)], axis=1), dtype)      # one matrix, as the mixers hold them
        gate = dev(rows(z, H * D), gdt)
        y = torch.empty((step.n_tokens, H * P), dtype=torch.float32, device="cuda")
        if form == "forget":
            ops32.channel_scan(qkv[:, :H * D], None, qkv[:, 2 * H * D:], H, D, P, gate, dev(bias), state, step, y, lower=dev(lower), q_act="silu")
        else:
            ops32.channel_scan(qkv[:, :H * D], qkv[:, H * D:2 * H * D], qkv[:, 2 * H * D:], H, D, P, gate, dev(bias), state, step, y, tau=tau,
                               q_scale=qs)
        return y.cpu().numpy()
    got, state = scan_in_portions(lengths, cuts, slots, ops32.scan_state_floats(H, D, P) + 5, call)
    for s in range(3):
        assert rel_err(got[s], want[s]) <= 3e-5, f"request {s}"
    state[0].zero_()
    again = call(state_step([lengths[1]], [0]), [1], {1: slice(0, lengths[1])}, state)
    assert rel_err(again, want[1]) <= 3e-5


def paged_rows(rng, lengths, kw, vw, page, dtype):
    """Random key rows [n, kw] and value rows [n, vw] of requests, scattered over pages in a random order."""
    blocks = [-(-n // page) for n in lengths]
    n_pages = sum(blocks) + 3
    perm = rng.permutation(n_pages)
    table = np.zeros((len(lengths), max(blocks) + 2), np.int32)
    kc, vc = np.full((n_pages * page, kw), 1e4, np.float32), np.full((n_pages * page, vw), -1e4, np.float32)   # stale rows hold large values
    ks, vs, at = [], [], 0
    for s, n in enumerate(lengths):
        k, v = rng.standard_normal((n, kw)).astype(np.float32), rng.standard_normal((n, vw)).astype(np.float32)
        for b in range(blocks[s]):
            pgn = perm[at]
            at += 1
            table[s, b] = pgn
            rows = slice(b * page, min((b + 1) * page, n))
            cnt = rows.stop - rows.start
            kc[pgn * page:pgn * page + cnt], vc[pgn * page:pgn * page + cnt] = k[rows], v[rows]
        ks.append(k)
        vs.append(v)
    cache = FakeCache(group=0, k=dev(kc, dtype), v=dev(to_value_layout(vc, page), dtype), page_tokens=page, window=0)
    return ks, vs, cache, ints(table)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,page,cap", [(4, 2, 16, 16, 16, 0.0), (3, 1, 32, 20, 8, 5.0), (8, 8, 64, 64, 16, 30.0), (6, 2, 48, 32, 4, 2.0),
                                               (6, 1, 40, 24, 16, 25.0), (2, 2, 10, 6, 8, 0.0), (4, 2, 128, 128, 16, 20.0), (6, 1, 32, 32, 8, 0.0),
                                               (8, 2, 64, 64, 32, 0.0), (16, 4, 96, 96, 16, 50.0)])
def test_attention_with_capped_scores_and_sigmoid_weights(ops32, dtype, H, G, D, Dv, page, cap):
    """Queries at the last positions of each request (a portion for some, a single token for others): every visible key
    weighs sigmoid(cap tanh(score / cap) + b_h), not normalised; a key far back, one at a page's last place and the
    query's own are made to stand out."""
    rng = np.random.default_rng(H * 100 + D + page)
    lengths, q_lens = [1, 5, 64, 130, 203], [1, 3, 64, 1, 17]
    ks, vs, cache, table = paged_rows(rng, lengths, G * D, G * Dv, page, dtype)
    bias = (rng.standard_normal(H) - 3.0).astype(np.float32)
    scale = 1.0 / math.sqrt(D)
    qs, positions, slots, wants = [], [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q = rng.standard_normal((n, H, D)).astype(np.float32)
        k, v = rounded(ks[s], dtype).reshape(n, G, D), rounded(vs[s], dtype).reshape(n, G, Dv)
        if n > 100:
            for far in (2, page - 1, n - 1):                # the last query of every head looks at these
                q[n - 1] += 3.0 * np.repeat(ks[s][far].reshape(G, D), H // G, axis=0) / math.sqrt(D) * 4.0 / 3.0
        qr = rounded(q, dtype)
        grp = np.arange(H) // (H // G)
        sc = np.einsum("ihd,jhd->hij", qr, k[:, grp]) * scale
        if cap:
            sc = cap * np.tanh(sc / cap)
        wgt = pg.sigmoid(sc + bias[:, None, None].astype(np.float64)) * np.tril(np.ones((n, n)))[None]
        full = np.einsum("hij,jhd->ihd", wgt, v[:, grp])
        qs.append(q[n - ql:])
        wants.append(full[n - ql:])
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = np.concatenate(qs).reshape(-1, H * D)
    want = np.concatenate(wants).reshape(-1, H * Dv)
    out = torch.empty((q.shape[0], H * Dv), dtype=dtype, device="cuda")
    step = FakeStep(ints(positions), ints(slots), table, None)
    ops32.paged_attention(dev(q, dtype), H, G, D, cache, step, 0, scale, out, v_head_dim=Dv, softcap=cap, weights="sigmoid", head_bias=dev(bias))
    err = np.max(np.abs(out.float().cpu().numpy() - want) / (np.abs(want) + 1.0))
    assert err <= (2e-5 if dtype == torch.float32 else 0.02), f"max |diff| {err:.3e}"
    # a cap alone, under the softmax
    if cap:
        s, n = 3, lengths[3]
        k, v = rounded(ks[s], dtype).reshape(n, G, D), rounded(vs[s], dtype).reshape(n, G, Dv)
        q1 = rounded(qs[s][-1:], dtype)
        grp = np.arange(H) // (H // G)
        sc = cap * np.tanh(np.einsum("ihd,jhd->hij", q1, k[:, grp]) * scale * 3.0 / cap)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        want1 = np.einsum("hij,jhd->ihd", p / p.sum(-1, keepdims=True), v[:, grp]).reshape(1, H * Dv)
        out1 = torch.empty((1, H * Dv), dtype=dtype, device="cuda")
        step1 = FakeStep(ints([n - 1]), ints([s]), table, None)
        ops32.paged_attention(dev(qs[s][-1:].reshape(1, H * D), dtype), H, G, D, cache, step1, 0, scale * 3.0, out1, v_head_dim=Dv, softcap=cap)
        assert np.max(np.abs(out1.float().cpu().numpy() - want1)) <= (2e-5 if dtype == torch.float32 else 0.02)


@pytest.mark.parametrize("H,G,D,page,cap,lengths,q_lens", [
    (8, 2, 64, 16, 30.0, [700, 1500], [1, 1]),              # single tokens: the keys cut into chunks, the chunks' sums added
    (16, 4, 128, 16, 0.0, [3000, 40, 1], [1, 1, 1]),
    (4, 1, 32, 8, 10.0, [1500], [64]),                      # a portion far into a prompt: few blocks, each cut into chunks
    (8, 4, 64, 16, 30.0, [900, 333], [900, 333]),           # whole prompts
    (8, 2, 128, 64, 5.0, [1100, 17], [300, 17]),
])
def test_sigmoid_weights_on_the_matrix_cores_at_long_contexts(ops16, H, G, D, page, cap, lengths, q_lens):
    """The matrix-core kernels' own cuttings (key chunks for few queries, four waves a tile for portions) against the
    plain kernel on the same cache, and against float64 for the last token of each request."""
    rng = np.random.default_rng(H + D + sum(lengths))
    ks, vs, cache, table = paged_rows(rng, lengths, G * D, G * D, page, torch.bfloat16)
    bias = (rng.standard_normal(H) - 4.0).astype(np.float32)
    scale = 1.0 / math.sqrt(D)
    qs, positions, slots = [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q = rng.standard_normal((ql, H, D)).astype(np.float32)
        if n > 100:
            q[-1] += 4.0 * np.repeat(ks[s][2].reshape(G, D), H // G, axis=0) / math.sqrt(D)      # a key far back stands out
        qs.append(q)
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = dev(np.concatenate(qs).reshape(-1, H * D), torch.bfloat16)
    step = FakeStep(ints(positions), ints(slots), table, None)
    out, other = torch.empty_like(q), torch.empty_like(q)
    args = dict(softcap=cap, weights="sigmoid", head_bias=dev(bias))
    ops16.paged_attention(q, H, G, D, cache, step, 0, scale, out, **args)
    ops16.force_plain_attention = True
    try:
        ops16.paged_attention(q, H, G, D, cache, step, 0, scale, other, **args)
    finally:
        ops16.force_plain_attention = False
    got, plain_got = out.float().cpu().numpy(), other.float().cpu().numpy()
    assert np.max(np.abs(got - plain_got) / (np.abs(plain_got) + 1.0)) <= 0.03            # (probabilities rounded to bf16 on the matrix cores)
    grp = np.arange(H) // (H // G)
    at = 0
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        at += ql
        k, v = rounded(ks[s], torch.bfloat16).reshape(n, G, D), rounded(vs[s], torch.bfloat16).reshape(n, G, D)
        sc = np.einsum("hd,jhd->hj", rounded(qs[s][-1], torch.bfloat16), k[:, grp]) * scale
        if cap:
            sc = cap * np.tanh(sc / cap)
        want = np.einsum("hj,jhd->hd", pg.sigmoid(sc + bias[:, None].astype(np.float64)), v[:, grp]).reshape(-1)
        assert np.max(np.abs(got[at - 1] - want) / (np.abs(want) + 1.0)) <= 0.02, f"request {s}"


@pytest.mark.parametrize("H,DK,C,page,lengths,q_lens", [
    (4, 128, 96, 16, [1, 5, 64, 130, 203], [1, 3, 64, 1, 17]),
    (16, 576, 512, 16, [700, 1500], [1, 1]),                # single tokens: the keys cut into chunks
    (16, 576, 512, 16, [300, 77], [300, 77]),               # whole prompts
    (2, 128, 64, 8, [1100, 17, 2], [300, 17, 2]),
    (40, 96, 32, 4, [150, 1], [9, 1]),                      # more heads than a tile has columns
    (12, 320, 256, 32, [900], [33]),
    (1, 48, 32, 16, [70, 200], [70, 1]),
])
def test_many_heads_on_one_wide_key_value_head(ops16, H, DK, C, page, lengths, q_lens):
    """What attention through latents asks of the attention kernels: every head reads the same key rows (wider than the
    value rows). The matrix-core kernel against float64 and against the plain kernel on the same cache; the last query of
    each long request is made to look at a key far back and at one at a page's last place."""
    rng = np.random.default_rng(H + DK + sum(lengths))
    ks, vs, cache, table = paged_rows(rng, lengths, DK, C, page, torch.bfloat16)
    scale = 1.0 / math.sqrt(DK)
    qs, positions, slots = [], [], []
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        q = rng.standard_normal((ql, H, DK)).astype(np.float32)
        if n > 100:
            q[-1] += 5.0 * (ks[s][2] + ks[s][page - 1])[None, :] / math.sqrt(DK)
        qs.append(q)
        positions += list(range(n - ql, n))
        slots += [s] * ql
    q = dev(np.concatenate(qs).reshape(-1, H * DK), torch.bfloat16)
    step = FakeStep(ints(positions), ints(slots), table, None)
    out = torch.empty((q.shape[0], H * C), dtype=torch.bfloat16, device="cuda")
    other = torch.empty_like(out)
    ops16.paged_attention(q, H, 1, DK, cache, step, 0, scale, out, v_head_dim=C)
    ops16.force_plain_attention = True
    try:
        ops16.paged_attention(q, H, 1, DK, cache, step, 0, scale, other, v_head_dim=C)
    finally:
        ops16.force_plain_attention = False
    got, plain_got = out.float().cpu().numpy(), other.float().cpu().numpy()
    assert np.max(np.abs(got - plain_got)) <= 0.03
    at = 0
    for s, (n, ql) in enumerate(zip(lengths, q_lens)):
        k, v = rounded(ks[s], torch.bfloat16), rounded(vs[s], torch.bfloat16)
        for i in sorted({0, ql // 2, ql - 1}):
            p_ = n - ql + i
            sc = (rounded(qs[s][i], torch.bfloat16) @ k[:p_ + 1].T) * scale
            pr = np.exp(sc - sc.max(-1, keepdims=True))
            want = ((pr / pr.sum(-1, keepdims=True)) @ v[:p_ + 1]).reshape(-1)
            assert np.max(np.abs(got[at + i] - want)) <= 0.03, f"request {s} token {i}"
        at += ql


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,R,C", [(3, 6, 4, 10), (1, 8, 8, 5), (4, 64, 64, 96), (2, 32, 64, 64), (16, 128, 64, 512)])
def test_rows_for_attention_through_latents(ops32, dtype, H, D, R, C):
    rng = np.random.default_rng(H + D + C)
    T = 11
    down = (rng.standard_normal((T, C + R)) * rng.uniform(0.1, 9.0, (T, 1))).astype(np.float32)
    q = rounded(rng.standard_normal((T, H * (D + R))), dtype)
    w = (1.0 + 0.2 * rng.standard_normal(C)).astype(np.float32)
    HD = R + C
    packed = torch.full((T, H * HD + HD + C + 3), 7.0, dtype=dtype, device="cuda")
    wide = dev(np.concatenate([np.zeros((T, 2), np.float32), down], axis=1))
    ops32.latent_pack(wide[:, 2:], dev(q, dtype), dev(w), 1e-5, packed, H, D, R, C)
    got = packed.float().cpu().numpy()
    c = pg.rms_norm(down[:, :C].astype(np.float64), w, 1e-5)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    for hd in range(H):
        assert np.array_equal(got[:, hd * HD:hd * HD + R], q[:, hd * (D + R) + D:(hd + 1) * (D + R)].astype(np.float32))
        assert np.all(got[:, hd * HD + R:(hd + 1) * HD] == 7.0)                                  # left for the folded queries
    key = got[:, H * HD:]
    assert np.max(np.abs(key[:, :R] - rounded(down[:, C:], dtype))) == 0.0
    assert np.max(np.abs(key[:, R:HD] - c) / (np.abs(c) + 1.0)) <= tol and np.array_equal(key[:, R:HD], key[:, HD:HD + C])
    assert np.all(key[:, HD + C:] == 7.0)


@pytest.mark.parametrize("E,top", [(5, 2), (10, 2), (4, 1), (3, 3), (64, 8), (256, 6)])
def test_router_with_the_softmax_over_the_chosen(ops32, E, top):
    rng = np.random.default_rng(E + top)
    T = 37
    z = (rng.standard_normal((T, E)) * 3.0).astype(np.float32)
    z[3] -= 200.0                                          # far from zero: the softmax takes the largest logit off first
    z[4, :2] = z[4].max() + 1.0                            # equal logits: the lower index first
    ids, wts = ops32.moe_route(dev(z), top, 1, 1, "softmax_chosen", True, 1.0)
    w = {"router": np.eye(E), "router.b": np.zeros(E)}
    want_ids, want_w = pg.route(z.astype(np.float64), w, "", top)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.max(np.abs(wts.cpu().numpy() - want_w)) <= 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,F,E,top,T", [(40, 12, 5, 3, 9), (40, 32, 3, 3, 4), (256, 64, 8, 2, 70), (256, 96, 6, 3, 300), (128, 64, 10, 2, 1)])
def test_gated_experts_weighted_on_their_output(ops32, ops16, dtype, W, F, E, top, T):
    """sum_e c_e Wdown_e (silu(Wgate_e h) * (Wup_e h)): the weight multiplies an expert's result, not its input."""
    ops = ops32 if dtype == torch.float32 else ops16
    rng = np.random.default_rng(W + F + T)
    h = rounded(rng.standard_normal((T, W)), dtype)
    gate, up = rounded(rng.standard_normal((E, F, W)) / math.sqrt(W), dtype), rounded(rng.standard_normal((E, F, W)) / math.sqrt(W), dtype)
    down = rounded(rng.standard_normal((E, W, F)) / math.sqrt(F), dtype)
    ids = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    wts = rng.uniform(0.05, 2.0, (T, top)).astype(np.float32)
    want = np.zeros((T, W))
    for t in range(T):
        for e, c in zip(ids[t], wts[t]):
            want[t] += c * (down[e] @ (pg.silu(gate[e] @ h[t]) * (up[e] @ h[t])))
    inter = F % 32 == 0
    wu = ops.interleave_experts(dev(gate, dtype), dev(up, dtype)) if inter else torch.cat([dev(gate, dtype), dev(up, dtype)], 1).contiguous()
    x0 = rng.standard_normal((T, W)).astype(np.float32)
    x = dev(x0)
    ops.moe_experts(dev(h, dtype), ints(ids), dev(wts), wu, dev(down, dtype), "relu2", x, gated=(1.0, 0.0, 0.0, inter), weight_on="output")
    err = np.max(np.abs(x.cpu().numpy() - x0 - want)) / np.max(np.abs(want))
    assert err <= (2e-5 if dtype == torch.float32 else 2e-2), f"{err:.3e}"


# ---- whole models ---------------------------------------------------------------------------------------------------

LENGTHS = {"small": [1, 2, 3, 23, 24, 57, 130], "cores": [3, 48, 49, 97, 161, 230]}


@pytest.fixture(scope="module", params=["small", "cores"])
def tiny(request, tmp_path_factory):
    name = request.param
    cfg = gh.CONFIGS[name]
    d = gh.make_model_dir(str(tmp_path_factory.mktemp("gitasun_" + name)), cfg, seed=len(name), stored=gh.STORED[name])
    reqs = gh.random_requests(cfg, LENGTHS[name], seed=7)
    return name, cfg, d, reqs, gh.plain_logits(d, reqs)


def engine_for(model_dir, dtype, name, max_tokens, max_seqs=4, graphs=True):
    import hf_cpu_amd
    return hf_cpu_amd.load_engine(model_dir, dtype=dtype, page_tokens=gh.PAGE[name], max_tokens=max_tokens, max_seqs=max_seqs, graphs=graphs)


def run_against_plain(name, d, reqs, want, dtype, steps, what, graphs=True):
    engine = engine_for(d, dtype, name, helpers.max_live_tokens(steps), graphs=graphs)
    got = helpers.run_trace_in_engine(engine, steps)
    worst = compare_for(dtype, got, want, TOL_OF.get((name, dtype), TOL[dtype]), what)
    engine.manager.check()
    assert not engine.manager.held and all(p.n_held == 0 for p in engine.manager.pools)
    return engine, got, worst


def test_the_stream_after_every_layer(gpu, tiny):
    """Layer by layer in fp32: the stream after each layer of a prompt against the plain implementation's."""
    from hf_cpu_amd.parts.block import PreNormBlock
    name, cfg, d, reqs, _ = tiny
    toks = reqs["r3"]
    pcfg, w = pg.read_model(d)
    want = []
    pg.forward(pcfg, w, toks, layers_out=want)
    engine = engine_for(d, "float32", name, 256, graphs=False)
    caught, orig = [], PreNormBlock.forward

    def fwd(self, ops, step, x, parts, caches, write_cache=True):
        orig(self, ops, step, x, parts, caches, write_cache)
        ops.settle()
        caught.append(x.clone())
    PreNormBlock.forward = fwd
    try:
        engine.step([("a", toks, [len(toks) - 1])])
    finally:
        PreNormBlock.forward = orig
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
    pcfg, w = pg.read_model(d)
    s = S.Session(d, dtype="float32", ctx_max=256, batch=16, page_size=gh.PAGE[name], max_seqs=4)
    gens = s.generate(prompts, temp=0.0, max_tokens=20)
    for g, p in zip(gens, prompts):
        assert len(g.tokens) == 20
        toks = list(p)
        for i, t in enumerate(g.tokens):
            row = pg.forward(pcfg, w, toks)[-1]
            assert row[int(np.argmax(row))] - row[t] <= 1e-4 * max(1.0, float(np.max(np.abs(row)))), \
                f"token {i} = {t}, plain picks {int(np.argmax(row))}"
            toks.append(t)


def test_command_line_generates_and_forks(gpu, tiny):
    """bin/hfamd on a folder of this design: greedy tokens are the plain implementation's; two continuations of one prompt
    (the second forks the first's pages and state rows after the prompt) drawn with seeds of their own start from the same
    logits; sampled runs with one seed repeat themselves."""
    import os
    import subprocess
    import sys
    name, cfg, d, reqs, _ = tiny
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = reqs["r3"]

    def run(extra):
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "hfamd"), "--stdin-mode", "none", "--model", d, "--dtype", "float32",
                            "--ctx-max", "128", "--page-size", str(gh.PAGE[name]), "--max-seqs", "4", "--log-level", "error",
                            "--prompt-ids", " ".join(map(str, prompt))] + extra, text=True, capture_output=True, timeout=300)
        assert r.returncode == 0, r.stderr
        toks = {}
        for line in r.stdout.replace("\x1e", "\n").splitlines():
            if line.startswith("@token "):
                f = dict(x.split("=", 1) for x in line.split(" ")[1:] if "=" in x)
                toks.setdefault(f.get("seq", "0"), []).append(int(f["id"]))
        return toks
    greedy = run(["--temp", "0", "--max-tokens", "6"])["0"]
    pcfg, w = pg.read_model(d)
    toks = list(prompt)
    for t in greedy:
        row = pg.forward(pcfg, w, toks)[-1]
        assert row[int(np.argmax(row))] - row[t] <= 1e-4 * max(1.0, float(np.max(np.abs(row))))
        toks.append(t)
    both = run(["--temp", "0", "--max-tokens", "5", "--n", "2"])
    assert both["0"] == greedy[:5] and both["1"] == greedy[:5]
    drawn = run(["--temp", "0.9", "--seed", "11", "--max-tokens", "8", "--n", "2"])
    again = run(["--temp", "0.9", "--seed", "11", "--max-tokens", "8", "--n", "2"])
    assert drawn == again and len(drawn["0"]) == 8 and len(drawn["1"]) == 8


def far_key_model(kind):
    """One layer whose attention is made to look far back. The norm's output has (nearly) the stream's direction, the table's
    last two columns are zero but for token 1, whose entry in the column before the last is large, and for a constant last
    column. Queries are a fixed vector u times that constant column; token 1's key is a large multiple of u: every query
    gives (nearly) all its weight to token 1's key, however far back; without token 1 in the prompt the weights are spread."""
    E = 64
    rng = np.random.default_rng(5)
    if kind == "latent":
        cfg = gh.config(50, E, [gh.layer(gh.latent(2, 16, 8, 16, 24, 12, scale=1.0), None)], embedding_scale=1.0)
        w = gh.make_weights(cfg, seed=1)
        p = "l0.mix."
        # the key's latent carries token 1's mark in its first coordinate; the queries' folded form reads it
        w[p + "dkv"][0] = 0.0
        w[p + "dkv"][0, E - 2] = 4.0
        w[p + "dkv.norm"][:] = 1.0
        w[p + "uk"][:, 0] = helpers.bf16_round(np.abs(rng.standard_normal(32)) + 1.0)
        w[p + "dq"][:] = 0.0
        w[p + "dq"][:, E - 1] = 1.0
        w[p + "dq.norm"][:] = 1.0
        w[p + "uq"][:] = 0.0
        for hd in range(2):
            w[p + "uq"][hd * 24:hd * 24 + 16] = helpers.bf16_round(np.abs(rng.standard_normal((16, 12))) * 0.1)
    else:
        cfg = gh.config(50, E, [gh.layer(gh.parallel(gh.left(2, 1, 32, 32, 8, scale=1.0, softcap=40.0), gh.right(1, 32, 32, 4.0), 1.0, 1.0), None)],
                        embedding_scale=1.0)
        w = gh.make_weights(cfg, seed=1)
        p = "l0.mix.left."
        u = np.zeros(32, np.float32)
        u[8:] = helpers.bf16_round(rng.standard_normal(24))          # in the part that is not rotated
        w[p + "q"][:], w[p + "q.b"][:], w[p + "k.b"][:] = 0.0, 0.0, 0.0
        w[p + "q"][:32, E - 1], w[p + "q"][32:, E - 1] = u, u
        w[p + "k"][:, E - 2] = 2.0 * u
        w[p + "pb"][:] = -20.0                                        # only a key that stands out weighs anything
        w["l0.mix.right.o"] = np.zeros_like(w["l0.mix.right.o"])
    w["embed"][:, E - 2:] = 0.0
    w["embed"][:, E - 1] = 1.0
    w["embed"][1, E - 2] = 30.0
    w["l0.norm1"] = np.float32(1.0)
    return cfg, w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["latent", "sigmoid"])
def test_a_key_far_back_among_hundreds(gpu, tmp_path, dtype, kind):
    """A prompt of 900 tokens in two portions and 20 decoded tokens: the marked token stands at position 2, at the last
    place of a page, or nowhere; the plain logits of the late tokens differ widely between these, and the engine's are the
    plain ones in each."""
    import hf_cpu_amd
    cfg, w = far_key_model(kind)
    d = gh.make_model_dir(str(tmp_path / "m"), cfg, seed=0, weights=w, stored="BF16")
    rng = np.random.default_rng(9)
    base = [int(t) for t in rng.integers(2, cfg["vocab"], 920)]
    reqs = {"none": base, "early": base[:2] + [1] + base[3:], "edge": base[:15] + [1] + base[16:]}
    want = gh.plain_logits(d, reqs)
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
    compare_for(dtype, got, want, TOL[dtype], f"far key {kind} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_decoded_token_by_token(gpu, tmp_path, dtype):
    """Two requests of 700 and 1,300 tokens: the prompt in two portions (the second begins in the middle of a page),
    then 45 tokens decoded together; attention cuts the keys of a decoded token over many waves, the states have been
    carried over a thousand steps."""
    import hf_cpu_amd
    cfg = gh.config(300, 128, residual_mult=0.85, layers=[
        gh.layer(gh.latent(4, 32, 32, 32, 64, 48), gh.dense(128)),
        gh.layer(gh.hgrn2(2, 64, 64), None),
        gh.layer(gh.parallel(gh.left(4, 2, 32, 32, 16, scaling=(6.0, 1.0, 3.0, 256), softcap=25.0), gh.right(2, 32, 64, 12.0), 0.8, 1.3), gh.moe(4, 2, 32, shared=32)),
        gh.layer(gh.hgrn2(2, 32, 64), gh.dense(96))])
    d = gh.make_model_dir(str(tmp_path / "m"), cfg, seed=4, stored="BF16")
    reqs = gh.random_requests(cfg, [700, 1300], seed=2)
    want = gh.plain_logits(d, reqs)
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
    compare_for(dtype, got, want, 2e-4 if dtype == "float32" else TOL[dtype], f"long prompts {dtype}")
    engine.manager.check()


def test_graphs_of_decode_steps_survive_a_longer_prompt(gpu, tmp_path):
    """Decode steps of a short request are captured into graphs; then a prompt arrives that is longer than anything before
    (work buffers and the table of heads behind the heads' grouped products grow); the short request's next steps, replayed
    or captured anew, still give the plain logits."""
    import hf_cpu_amd
    cfg = gh.config(120, 64, residual_mult=0.9, layers=[gh.layer(gh.latent(4, 16, 16, 16, 48, 24), gh.dense(64)),
                                                        gh.layer(gh.hgrn2(2, 16, 16), None)])
    d = gh.make_model_dir(str(tmp_path / "m"), cfg, seed=2, stored="BF16")
    reqs = gh.random_requests(cfg, [40, 1300], seed=5)
    want = gh.plain_logits(d, reqs)
    a, b = reqs["r0"], reqs["r1"]
    steps = [helpers._step(0, [("r0", a[:20], [19])])]
    steps += [helpers._step(len(steps) + i, [("r0", a[20 + i:21 + i], [0])]) for i in range(8)]
    steps.append(helpers._step(len(steps), [("r1", b, [0, 1299])], ["r1"]))
    steps += [helpers._step(len(steps) + i, [("r0", a[28 + i:29 + i], [0])], ["r0"] if i == 11 else []) for i in range(12)]
    for dtype in ("float32", "bfloat16"):
        engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=helpers.max_live_tokens(steps), max_seqs=2)
        got = helpers.run_trace_in_engine(engine, steps)
        assert engine.graph_replays > 0
        compare_for(dtype, got, want, TOL[dtype], f"graphs and a longer prompt {dtype}")


def test_random_weights_and_other_orders_of_layers(gpu, tmp_path):
    """``write_random_model`` makes a folder for this design too (the latents' and the decay's inner sizes from the
    configuration), and the engine reads it back: a model of one recurrence, one of one side-by-side layer with a single
    head everywhere, and one with widths that are no multiple of 8."""
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    one = gh.config(90, 64, [gh.layer(gh.hgrn2(1, 32, 32), gh.dense(16))])
    two = gh.config(90, 64, [gh.layer(gh.parallel(gh.left(1, 1, 32, 32, 32), dict(gh.right(1, 32, 32, 2.0), decay_rank=4)), None)])
    odd = gh.config(77, 100, eps=1e-3, residual_mult=0.9, layers=[
        gh.layer(gh.parallel(gh.left(3, 1, 20, 28, 10), dict(gh.right(4, 5, 3, 8.0), decay_rank=3)), gh.moe(3, 2, 12, shared=5)),
        gh.layer(gh.latent(5, 4, 2, 3, 9, 6), None),
        gh.layer(gh.hgrn2(2, 9, 7), gh.dense(20))])
    for k, c in enumerate((one, two, odd)):
        d = str(tmp_path / f"m{k}")
        hf_cpu_amd.write_random_model(d, config_from_dict(c), seed=3, dtype="bfloat16")
        pcfg, w = pg.read_model(d)
        toks = [int(t) for t in np.random.default_rng(0).integers(0, c["vocab"], 45)]
        want = pg.forward(pcfg, w, toks)
        for dtype in ("float32", "bfloat16"):
            engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=4, max_tokens=64, max_seqs=1)
            got = engine.step([("a", toks[:31], list(range(31)))]).cpu().numpy()
            rows = {("a", i): row for i, row in enumerate(got)}
            for i in range(31, 45):
                rows[("a", i)] = engine.step([("a", toks[i:i + 1], [0])]).cpu().numpy()[0]
            compare_for(dtype, rows, {"a": want}, TOL[dtype] if dtype == "float32" else 8e-2, f"random weights {k} {dtype}")


@pytest.mark.parametrize("seed", range(6))
def test_configurations_drawn_at_random(gpu, tmp_path, seed):
    """Layers of every kind in any order with sizes drawn at random (even seeds: sizes for the matrix cores): a prompt, a
    portion that starts in the middle of a page, then single tokens, in fp32 and in bf16."""
    import hf_cpu_amd
    rng = np.random.default_rng(100 + seed)
    cfg = gh.random_config(rng, big=seed % 2 == 0)
    d = gh.make_model_dir(str(tmp_path / "m"), cfg, seed=seed, stored="BF16" if seed % 2 == 0 else "F32")
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 110)]
    pcfg, w = pg.read_model(d)
    want = pg.forward(pcfg, w, toks)
    steps = [helpers._step(0, [("a", toks[:55], range(55))]), helpers._step(1, [("a", toks[55:88], range(33))])]
    steps += [helpers._step(2 + i, [("a", toks[88 + i:89 + i], [0])], ["a"] if i == 21 else []) for i in range(22)]
    for dtype in ("float32", "bfloat16"):
        engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=16, max_tokens=128, max_seqs=2, graphs=dtype == "float32")
        got = helpers.run_trace_in_engine(engine, steps)
        compare_for(dtype, got, {"a": want}, TOL[dtype] if dtype == "float32" else 8e-2, f"random configuration {seed} {dtype}: {cfg}")
