// Mixers with per-request state of fixed size: a short causal convolution whose last inputs are carried from step to
// step, and a linear recurrence over a matrix state per head (state-space layers, linear attention).
//
//   hfa_causal_conv   out[t, c] = act(bias[c] + sum_j taps[c, j] in[t - (K - 1) + j, c]) per channel, the K - 1 inputs
//                     before a request's first token of this step taken from its state row, which then receives the
//                     last K - 1 inputs of the step
//   hfa_linear_scan   S <- a_t S + k_t (b_t v_t)^T, y_t = S^T q_t + d v_t per (request, head), S in fp32 in the state row
//   hfa_delta_scan    S <- g_t * S (a decay per row), u = beta_t (v_t - S^T k_t), S <- S + k_t u^T, y_t = S^T q_t
//
// Both walk a request's tokens of the step in order from the state that the step before left, so a token's result
// does not depend on where a prompt was cut or on what else the step holds.
#include "api.h"
#include "common.h"

#define CONV_MAX_TAPS 8
#define CONV_SEG 64              // tokens that one thread walks

// One thread a (request, run of CONV_SEG tokens, channel). state row: [K - 1][C] inputs, oldest first.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ in, int ld_in, const float* __restrict__ taps,
                                                         const float* __restrict__ bias, int C, int K,
                                                         float* __restrict__ state, size_t state_ld,
                                                         const int* __restrict__ q_start, const int* __restrict__ seq_slot,
                                                         float* __restrict__ out, int ldo, int act) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.z;
    if (c >= C) return;
    const int q0 = q_start[s], n = q_start[s + 1] - q0, t0 = blockIdx.y * CONV_SEG;
    if (t0 >= n) return;
    float* st = state + (size_t)seq_slot[s] * state_ld;
    // the input at place i of the request's tokens of this step; i < 0 reaches into the state
    auto input = [&](int i) { return i >= 0 ? to_f32(in[(size_t)(q0 + i) * ld_in + c]) : st[(size_t)(K - 1 + i) * C + c]; };
    float w[CONV_MAX_TAPS], win[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; j++) {
        w[j] = j < K ? taps[(size_t)c * K + j] : 0.f;
        win[j] = j < K - 1 ? input(t0 - (K - 1) + j) : 0.f;
    }
    if (t0 == 0) {
        // The only thread that reads this channel's state is also the one that writes it: all reads come first.
        float next[CONV_MAX_TAPS];
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; j++) next[j] = j < K - 1 ? input(n - (K - 1) + j) : 0.f;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; j++)
            if (j < K - 1) st[(size_t)j * C + c] = next[j];
    }
    const float b = bias ? bias[c] : 0.f;
    const int t1 = t0 + CONV_SEG < n ? t0 + CONV_SEG : n;
    for (int t = t0; t < t1; t++) {
        win[K - 1] = to_f32(in[(size_t)(q0 + t) * ld_in + c]);
        float acc = b;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; j++)
            if (j < K) acc = fmaf(w[j], win[j], acc);
        out[(size_t)(q0 + t) * ldo + c] = act == HFA_ACT_SILU ? acc / (1.0f + expf(-acc)) : acc;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS - 1; j++) win[j] = win[j + 1];
    }
}

extern "C" int hfa_causal_conv(const void* in, int dtype, int ld_in, const float* taps, const float* bias, int n_channels,
                               int n_taps, float* state, size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs,
                               int max_q_len, float* out, int ldo, int act, hipStream_t stream) {
    HFA_REQUIRE(in && taps && (state || n_taps == 1) && q_start && seq_slot && out && n_channels > 0 && n_seqs > 0 && max_q_len > 0,
                "causal_conv: bad arguments");
    HFA_REQUIRE(n_taps >= 1 && n_taps <= CONV_MAX_TAPS, "causal_conv: %d taps (1 to %d)", n_taps, CONV_MAX_TAPS);
    HFA_REQUIRE(ld_in >= n_channels && ldo >= n_channels && state_ld >= (size_t)(n_taps - 1) * n_channels,
                "causal_conv: a row is shorter than its channels");
    HFA_REQUIRE(act == HFA_ACT_NONE || act == HFA_ACT_SILU, "causal_conv: the activation is silu or none");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "causal_conv: unknown dtype %d", dtype);
    HFA_REQUIRE(n_seqs <= 65535 && (max_q_len + CONV_SEG - 1) / CONV_SEG <= 65535, "causal_conv: the step exceeds the grid");
    dim3 grid((n_channels + 255) / 256, (max_q_len + CONV_SEG - 1) / CONV_SEG, n_seqs);
    if (dtype == HFA_F32)
        causal_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)in, ld_in, taps, bias, n_channels, n_taps, state, state_ld,
                                                            q_start, seq_slot, out, ldo, act);
    else
        causal_conv_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)in, ld_in, taps, bias, n_channels, n_taps, state, state_ld,
                                                           q_start, seq_slot, out, ldo, act);
    HFA_LAUNCH_CHECK("causal_conv");
    return 0;
}

// ---- the linear recurrence ------------------------------------------------------------------------------------
// A block of four waves owns 256 / NS columns p of one head's state S [N][P] of one request and walks the request's
// tokens in order. A column is spread over NS neighbouring lanes: lane ns holds S[n][p] for the NPT values n = ns NPT
// + i in registers for the whole walk, and a token's output is the sum over the NS lanes. The tokens' k, q, v, a and b
// are staged through LDS SCAN_TOKENS at a time; the next tokens' loads are on their way while these are walked. Inside
// the walk nothing crosses lanes: every lane leaves its share of a token's output in LDS, and after SCAN_TOKENS tokens
// the shares are added up (lane 0's first, in a fixed order) and the outputs leave as whole runs of columns, so the
// only chain from token to token is the one the recurrence itself has.
//
// In the state row a head's values lie in the order the lanes read them: value (n = ns NPT + i, p) of head h at
// (h NPT + i) * P_pad * NS + p * NS + ns, with P_pad = P rounded up to whole blocks and n padded to NS NPT (the
// padding stays zero): a wave reads and writes whole lines. NS and NPT follow from N alone (scan_shape), so every
// step finds the layout that the step before left; hfa_linear_scan_state_floats gives the size of a row.
//
// gate 0: a_t = decay[h], b_t = 1 (a fixed decay per head).
// gate 1: dt = softplus(step[t, h] + step_bias[h]), a_t = exp(-exp(a_log[h]) dt), b_t = dt (a step size per token).
// gate 2: exponential gates kept stable by a running maximum m (0 for a new request, kept beside the states): with
//         li = cap tanh((step[t, h] + step_bias[h]) / cap) and lf = logsigmoid(cap tanh((step2[t, h] + step_bias2[h]) / cap)),
//         m_t = max(lf + m_(t-1), li), a_t = exp(lf + m_(t-1) - m_t), b_t = exp(li - m_t). The state has one more column
//         whose value is 1 for every token, so that it holds n_t = a_t n_(t-1) + b_t k_t; its output n_t . q_t does not
//         leave as a column of y but as denom[t, h] = 1 / (max(|n_t . q_t|, exp(-m_t)) + 1e-6), by which the reader of y
//         multiplies the head's outputs. Every block of columns keeps a copy of m of its own (a block may start after
//         another of the same head has ended), behind the states: m_off + h * blocks + block.
#define SCAN_TOKENS 16
#define SCAN_THREADS 256

// Up to sixteen lanes a column with 4, 8 or 16 values each. (Four values a lane on up to 64 lanes a column, which puts
// four times the waves on a SIMD for states of 128 rows, was measured: a prompt of 2,048 tokens 17 % quicker at 64 heads,
// 50 % slower at 128 heads, decode steps of 64 requests 50 % slower: more blocks, each with the same staging and barriers.)
static void scan_shape(int N, int* ns, int* npt) {
    *ns = N >= 64 ? 16 : N > 16 ? 8 : 4;
    const int per = (N + *ns - 1) / *ns;
    *npt = per <= 4 ? 4 : per <= 8 ? 8 : 16;
}

extern "C" size_t hfa_linear_scan_state_floats(int n_heads, int qk_dim, int v_dim) {
    int ns, npt;
    scan_shape(qk_dim, &ns, &npt);
    const int pt = SCAN_THREADS / ns, p_pad = (v_dim + pt - 1) / pt * pt;
    return (size_t)n_heads * ns * npt * p_pad;
}

template <typename T, typename TS, int NS, int NPT>
__global__ __launch_bounds__(SCAN_THREADS) void linear_scan_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, int heads_per_qk, int N, const T* __restrict__ v,
    int ldv, int P, int gate, const float* __restrict__ decay, const TS* __restrict__ step, int ld_step,
    const float* __restrict__ step_bias, const float* __restrict__ a_log, const float* __restrict__ skip,
    float* __restrict__ state, size_t state_ld, const int* __restrict__ q_start, const int* __restrict__ seq_slot,
    float* __restrict__ y, int ldy, const TS* __restrict__ step2, const float* __restrict__ step_bias2, float cap, float q_scale,
    float* __restrict__ denom, size_t m_off) {
    constexpr int NPAD = NS * NPT, PT = SCAN_THREADS / NS, TOK = SCAN_TOKENS;
    constexpr int RK = TOK * NPAD / SCAN_THREADS, RV = (TOK * PT + SCAN_THREADS - 1) / SCAN_THREADS;
    static_assert(TOK * NPAD % SCAN_THREADS == 0 && NPT % 4 == 0, "the staging loops are whole");
    __shared__ __attribute__((aligned(16))) float k_s[TOK * NPAD];
    __shared__ __attribute__((aligned(16))) float q_s[TOK * NPAD];
    __shared__ float v_s[TOK * PT];
    __shared__ float a_s[TOK], b_s[TOK], m_s[TOK];
    __shared__ __attribute__((aligned(16))) float part_s[TOK * SCAN_THREADS];      // [token][column][lane of the column]
    const int h = blockIdx.x, s = blockIdx.y, pz = blockIdx.z, tid = threadIdx.x;
    const int pl = tid / NS, ns = tid % NS;
    const int q0 = q_start[s], n_tok = q_start[s + 1] - q0;
    if (n_tok <= 0) return;
    const int g = h / heads_per_qk, p_pad = (int)gridDim.z * PT;
    float* S = state + (size_t)seq_slot[s] * state_ld + (size_t)h * NPT * p_pad * NS + (size_t)pz * SCAN_THREADS + tid;
    float st[NPT];
#pragma unroll
    for (int i = 0; i < NPT; i++) st[i] = S[(size_t)i * p_pad * NS];
    const float d = skip ? skip[h] : 0.f;
    const float head_decay = gate == 0 ? decay[h] : 0.f;
    const float neg_rate = gate == 1 ? -expf(a_log[h]) : 0.f, sb = gate >= 1 ? step_bias[h] : 0.f;
    const float sb2 = gate == 2 ? step_bias2[h] : 0.f, inv_cap = gate == 2 ? 1.0f / cap : 0.f;
    float* m_at = state + (size_t)seq_slot[s] * state_ld + m_off + (size_t)h * gridDim.z + pz;
    float m_run = gate == 2 ? *m_at : 0.f;               // the running maximum, followed by the block's first wave
    const T* kg = k + (size_t)q0 * ldk + g * N;
    const T* qg = q + (size_t)q0 * ldq + g * N;
    const T* vg = v + (size_t)q0 * ldv + h * P + pz * PT;
    // Two sets of registers take turns: while one chunk of tokens is walked, the loads of the next two are on their way
    // (a trip to memory takes longer than the walk of one chunk).
    struct Staged { float k[RK], q[RK], v[RV], step, step2; };
    Staged set_a, set_b;
    // the tokens c0 .. c0 + TOK - 1 into registers (zeros beyond the request's tokens, beyond N and beyond P)
    auto fetch = [&](Staged& g_, int c0) {
        if (c0 >= n_tok) return;
#pragma unroll
        for (int r = 0; r < RK; r++) {
            const int idx = tid + r * SCAN_THREADS, t = c0 + idx / NPAD, n = idx % NPAD;
            const bool ok = t < n_tok && n < N;
            g_.k[r] = ok ? to_f32(kg[(size_t)t * ldk + n]) : 0.f;
            g_.q[r] = ok ? to_f32(qg[(size_t)t * ldq + n]) : 0.f;
        }
#pragma unroll
        for (int r = 0; r < RV; r++) {
            const int idx = tid + r * SCAN_THREADS, t = c0 + idx / PT, pp = idx % PT;
            g_.v[r] = (idx < TOK * PT && t < n_tok && pz * PT + pp < P) ? to_f32(vg[(size_t)t * ldv + pp]) : 0.f;
            if (gate == 2 && idx < TOK * PT && t < n_tok && pz * PT + pp == P) g_.v[r] = 1.f;       // the normaliser's column
        }
        g_.step = (gate >= 1 && tid < TOK && c0 + tid < n_tok) ? to_f32(step[(size_t)(q0 + c0 + tid) * ld_step + h]) : 0.f;
        g_.step2 = (gate == 2 && tid < TOK && c0 + tid < n_tok) ? to_f32(step2[(size_t)(q0 + c0 + tid) * ld_step + h]) : 0.f;
    };
    auto stash = [&](const Staged& g_, int c0) {
#pragma unroll
        for (int r = 0; r < RK; r++) {
            k_s[tid + r * SCAN_THREADS] = g_.k[r];
            q_s[tid + r * SCAN_THREADS] = g_.q[r] * q_scale;
        }
#pragma unroll
        for (int r = 0; r < RV; r++)
            if (tid + r * SCAN_THREADS < TOK * PT) v_s[tid + r * SCAN_THREADS] = g_.v[r];
        if (gate == 2) {
            if (tid < WAVE) {                                   // the maximum runs from token to token: one wave, in order
                const float li = cap * tanhf((g_.step + sb) * inv_cap), zf = cap * tanhf((g_.step2 + sb2) * inv_cap);
                const float lf = -(fmaxf(-zf, 0.f) + log1pf(expf(-fabsf(zf))));          // logsigmoid
                // only the maximum itself is a chain (an add and a maximum a token, the gates read from their lanes); the
                // exponentials wait until every lane knows its token's maximum and the one before
                float m_before = 0.f, m_mine = 0.f;
#pragma unroll
                for (int t = 0; t < TOK; t++) {
                    if (c0 + t < n_tok) {                           // (the same for the whole wave)
                        const float f_t = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lf), t));
                        const float i_t = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(li), t));
                        const float mn = fmaxf(f_t + m_run, i_t);
                        if (tid == t) { m_before = m_run; m_mine = mn; }
                        m_run = mn;
                    }
                }
                if (tid < TOK) {
                    const bool live = c0 + tid < n_tok;
                    a_s[tid] = live ? expf(lf + m_before - m_mine) : 0.f;
                    b_s[tid] = live ? expf(li - m_mine) : 0.f;
                    m_s[tid] = m_mine;
                }
            }
        } else if (tid < TOK) {
            if (gate == 1) {
                const float z = g_.step + sb;
                const float dt = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));          // softplus, exact for every z
                a_s[tid] = expf(neg_rate * dt);
                b_s[tid] = dt;
            } else {
                a_s[tid] = head_decay;
                b_s[tid] = 1.f;
            }
        }
    };
    auto chunk = [&](Staged& g_, int c0) {
        const int nt = n_tok - c0 < TOK ? n_tok - c0 : TOK;
        __syncthreads();                                   // the walk before has read what is overwritten now
        stash(g_, c0);
        __syncthreads();
        fetch(g_, c0 + 2 * TOK);
        // A token's operands leave LDS two tokens before (three gained nothing) its multiply-adds: the only chain from token to token is the
        // state's own, and a wave that has a SIMD to itself would otherwise wait for every read.
        struct Operands { float4 k[NPT / 4], q[NPT / 4]; float a, bv; };
        auto read = [&](int t, Operands& o) {
            const float4* kt = reinterpret_cast<const float4*>(k_s + t * NPAD + ns * NPT);
            const float4* qt = reinterpret_cast<const float4*>(q_s + t * NPAD + ns * NPT);
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                o.k[i] = kt[i];
                o.q[i] = qt[i];
            }
            o.a = a_s[t];
            o.bv = b_s[t] * v_s[t * PT + pl];
        };
        auto token = [&](int t, const Operands& o) {
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                const float4 kk = o.k[i], qq = o.q[i];
                st[4 * i] = fmaf(o.a, st[4 * i], kk.x * o.bv);
                st[4 * i + 1] = fmaf(o.a, st[4 * i + 1], kk.y * o.bv);
                st[4 * i + 2] = fmaf(o.a, st[4 * i + 2], kk.z * o.bv);
                st[4 * i + 3] = fmaf(o.a, st[4 * i + 3], kk.w * o.bv);
                acc0 = fmaf(st[4 * i], qq.x, acc0);
                acc1 = fmaf(st[4 * i + 1], qq.y, acc1);
                acc0 = fmaf(st[4 * i + 2], qq.z, acc0);
                acc1 = fmaf(st[4 * i + 3], qq.w, acc1);
            }
            part_s[t * SCAN_THREADS + tid] = acc0 + acc1;
        };
        if (nt == TOK) {
            Operands ring[3];
            read(0, ring[0]);
            read(1, ring[1]);
#pragma unroll
            for (int t = 0; t < TOK; t++) {
                if (t + 2 < TOK) read(t + 2, ring[(t + 2) % 3]);
                token(t, ring[t % 3]);
            }
        } else {
            for (int t = 0; t < nt; t++) {
                Operands o;
                read(t, o);
                token(t, o);
            }
        }
        __syncthreads();
        // the outputs of the tokens just walked: thread -> (token, column), the lanes' shares added in lane order
        for (int idx = tid; idx < nt * PT; idx += SCAN_THREADS) {
            const int t = idx / PT, pp = idx % PT;
            if (pz * PT + pp > P || (pz * PT + pp == P && gate != 2)) continue;
            const float4* sh = reinterpret_cast<const float4*>(part_s + t * SCAN_THREADS + pp * NS);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NS / 4; i++) {
                const float4 u = sh[i];
                acc = ((acc + u.x) + u.y) + u.z + u.w;
            }
            if (pz * PT + pp == P)
                denom[(size_t)(q0 + c0 + t) * gridDim.x + h] = 1.0f / (fmaxf(fabsf(acc), expf(-m_s[t])) + 1e-6f);
            else
                y[(size_t)(q0 + c0 + t) * ldy + h * P + pz * PT + pp] = fmaf(d, v_s[t * PT + pp], acc);
        }
    };
    fetch(set_a, 0);
    fetch(set_b, TOK);
    for (int c0 = 0; c0 < n_tok; c0 += 2 * TOK) {
        chunk(set_a, c0);
        if (c0 + TOK < n_tok) chunk(set_b, c0 + TOK);
    }
#pragma unroll
    for (int i = 0; i < NPT; i++) S[(size_t)i * p_pad * NS] = st[i];
    if (gate == 2 && tid == 0) *m_at = m_run;
}

extern "C" size_t hfa_linear_scan_max_floats(int n_heads, int qk_dim, int v_dim) {
    int ns, npt;
    scan_shape(qk_dim, &ns, &npt);
    const int pt = SCAN_THREADS / ns;
    return (size_t)n_heads * ((v_dim + 1 + pt - 1) / pt);
}

extern "C" int hfa_linear_scan(const void* q, int ldq, const void* k, int ldk, int qk_heads, int qk_dim, const void* v,
                               int ldv, int n_heads, int v_dim, int dtype, int gate, const float* decay, const void* step,
                               int step_dtype, int ld_step, const float* step_bias, const float* a_log, const float* skip,
                               float* state, size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs, float* y,
                               int ldy, const void* step2, const float* step_bias2, float cap, float q_scale, float* denom,
                               hipStream_t stream) {
    HFA_REQUIRE(q && k && v && state && q_start && seq_slot && y && n_seqs > 0, "linear_scan: a null argument");
    HFA_REQUIRE(n_heads > 0 && qk_heads > 0 && n_heads % qk_heads == 0 && qk_dim > 0 && v_dim > 0,
                "linear_scan: %d heads over %d heads of keys", n_heads, qk_heads);
    HFA_REQUIRE(qk_dim <= 256, "linear_scan: a state of %d rows a head is too large (at most 256)", qk_dim);
    HFA_REQUIRE(ldq >= qk_heads * qk_dim && ldk >= qk_heads * qk_dim && ldv >= n_heads * v_dim && ldy >= n_heads * v_dim &&
                    state_ld >= hfa_linear_scan_state_floats(n_heads, qk_dim, v_dim + (gate == 2 ? 1 : 0)) +
                                    (gate == 2 ? hfa_linear_scan_max_floats(n_heads, qk_dim, v_dim) : 0),
                "linear_scan: a row is shorter than its heads (a state row holds hfa_linear_scan_state_floats values; gate 2: "
                "those of one more column, and hfa_linear_scan_max_floats)");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "linear_scan: unknown dtype %d", dtype);
    HFA_REQUIRE((gate == 0 && decay) || (gate == 1 && step && step_bias && a_log && ld_step >= n_heads &&
                                         (step_dtype == HFA_F32 || step_dtype == HFA_BF16)) ||
                    (gate == 2 && step && step2 && step_bias && step_bias2 && denom && cap > 0.f && !skip && ld_step >= n_heads &&
                     (step_dtype == HFA_F32 || step_dtype == HFA_BF16)),
                "linear_scan: gate 0 needs a decay per head, gate 1 step sizes, their bias and the logarithm of the rate, gate 2 "
                "both gates' inputs and biases, a positive cap and a place for the denominators (and no skip)");
    int ns, npt;
    scan_shape(qk_dim, &ns, &npt);
    const int pt = SCAN_THREADS / ns, p_tiles = (v_dim + (gate == 2 ? 1 : 0) + pt - 1) / pt;
    const size_t m_off = hfa_linear_scan_state_floats(n_heads, qk_dim, v_dim + 1);
    HFA_REQUIRE(n_heads <= 65535 && n_seqs <= 65535 && p_tiles <= 65535, "linear_scan: the step exceeds the grid");
    dim3 grid(n_heads, n_seqs, p_tiles);
#define SCAN_GO(T, TS, NS, NPT)                                                                                          \
    linear_scan_kernel<T, TS, NS, NPT><<<grid, SCAN_THREADS, 0, stream>>>(                                               \
        (const T*)q, ldq, (const T*)k, ldk, n_heads / qk_heads, qk_dim, (const T*)v, ldv, v_dim, gate, decay, (const TS*)step, \
        ld_step, step_bias, a_log, skip, state, state_ld, q_start, seq_slot, y, ldy, (const TS*)step2, step_bias2, cap, q_scale, \
        denom, m_off)
#define SCAN_SIZES(T, TS)                                          \
    do {                                                           \
        if (ns == 4) SCAN_GO(T, TS, 4, 4);                         \
        else if (ns == 8 && npt == 4) SCAN_GO(T, TS, 8, 4);        \
        else if (ns == 8) SCAN_GO(T, TS, 8, 8);                    \
        else if (npt == 4) SCAN_GO(T, TS, 16, 4);                  \
        else if (npt == 8) SCAN_GO(T, TS, 16, 8);                  \
        else SCAN_GO(T, TS, 16, 16);                               \
    } while (0)
    if (dtype == HFA_F32) { if (step_dtype == HFA_BF16 && gate >= 1) SCAN_SIZES(float, bf16); else SCAN_SIZES(float, float); }
    else { if (step_dtype == HFA_F32 && gate >= 1) SCAN_SIZES(bf16, float); else SCAN_SIZES(bf16, bf16); }
#undef SCAN_SIZES
#undef SCAN_GO
    HFA_LAUNCH_CHECK("linear_scan");
    return 0;
}

// ---- the gated delta rule ----------------------------------------------------------------------------------------------
// Per head h (queries and keys of head h / (n_heads / qk_heads)), S [N][P] in the state row, in hfa_linear_scan's layout:
//   g_t[n] = exp(-exp(a_log[h]) softplus(a[t, h N + n] + dt_bias[h N + n]))        a decay per key channel (row of S)
//   S <- g_t * S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  y_t = S^T q_t     beta_t = sigmoid(b[t, h])
// with k_t and q_t made unit vectors first (x / sqrt(sum x^2 + unit_eps)) and q_t times q_scale. All inputs, the state
// and every operation are fp32. The block, its lanes and the staging through LDS are linear_scan_kernel's; what differs is
// that a token's correction needs S^T k_t whole before the state moves, so the lanes of a column add their shares of it
// across lanes inside the walk (a butterfly: every lane gets the same bits), where that kernel has no traffic at all.
// The sum over an aligned run of NS neighbouring lanes (4, 8 or 16: inside a row of the data-parallel primitives), left in
// every lane of the run with the same bits: neighbours, pairs, then the mirror of a half row and of a row, which pair a
// lane with one of the other quad or half whose lanes all hold that side's sum already. No trip through LDS: these are
// modifiers of the adds themselves, and they stand in the chain from one token's state to the next.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
template <int NS>
__device__ __forceinline__ float run_sum(float x) {
    if constexpr (NS == 4 || NS == 8 || NS == 16) {
        x += dpp_move<0xB1>(x);                            // quad_perm [1, 0, 3, 2]
        x += dpp_move<0x4E>(x);                            // quad_perm [2, 3, 0, 1]
        if constexpr (NS >= 8) x += dpp_move<0x141>(x);    // row_half_mirror
        if constexpr (NS >= 16) x += dpp_move<0x140>(x);   // row_mirror
    } else {
#pragma unroll
        for (int off = 1; off < NS; off <<= 1) x += __shfl_xor(x, off, WAVE);
    }
    return x;
}

// AHEAD: the walk of whole chunks reads operands ahead (steps with prompt portions); without it the kernel needs fewer
// registers and more blocks share a compute unit, which is what a step of single tokens lives on.
template <int NS, int NPT, bool AHEAD>
__global__ __launch_bounds__(SCAN_THREADS) void delta_scan_kernel(
    const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, int heads_per_qk, int N, const float* __restrict__ v,
    int ldv, int P, const float* __restrict__ a, int lda, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const float* __restrict__ b, int ldb, float q_scale, float unit_eps, float* __restrict__ state, size_t state_ld,
    const int* __restrict__ q_start, const int* __restrict__ seq_slot, float* __restrict__ y, int ldy) {
    constexpr int NPAD = NS * NPT, PT = SCAN_THREADS / NS, TOK = SCAN_TOKENS;
    constexpr int RK = TOK * NPAD / SCAN_THREADS, RV = (TOK * PT + SCAN_THREADS - 1) / SCAN_THREADS;
    static_assert(TOK * NPAD % SCAN_THREADS == 0 && NPT % 4 == 0, "the staging loops are whole");
    __shared__ __attribute__((aligned(16))) float k_s[TOK * NPAD];
    __shared__ __attribute__((aligned(16))) float q_s[TOK * NPAD];
    __shared__ __attribute__((aligned(16))) float g_s[TOK * NPAD];
    __shared__ float v_s[TOK * PT];
    __shared__ float b_s[TOK];
    __shared__ __attribute__((aligned(16))) float part_s[TOK * SCAN_THREADS];
    const int h = blockIdx.x, s = blockIdx.y, pz = blockIdx.z, tid = threadIdx.x;
    const int pl = tid / NS, ns = tid % NS, lane = tid & (WAVE - 1), wv = tid / WAVE;
    const int q0 = q_start[s], n_tok = q_start[s + 1] - q0;
    if (n_tok <= 0) return;
    const int g = h / heads_per_qk, p_pad = (int)gridDim.z * PT;
    float* S = state + (size_t)seq_slot[s] * state_ld + (size_t)h * NPT * p_pad * NS + (size_t)pz * SCAN_THREADS + tid;
    float st[NPT];
#pragma unroll
    for (int i = 0; i < NPT; i++) st[i] = S[(size_t)i * p_pad * NS];
    const float neg_rate = -expf(a_log[h]);
    const float* kg = k + (size_t)q0 * ldk + g * N;
    const float* qg = q + (size_t)q0 * ldq + g * N;
    const float* ag = a + (size_t)q0 * lda + h * N;
    const float* vg = v + (size_t)q0 * ldv + h * P + pz * PT;
    float bias_r[RK];                                      // the decay's bias of the channels this thread stages
#pragma unroll
    for (int r = 0; r < RK; r++) {
        const int n = (tid + r * SCAN_THREADS) % NPAD;
        bias_r[r] = n < N ? dt_bias[h * N + n] : 0.f;
    }
    struct Staged { float k[RK], q[RK], a[RK], v[RV], b; };
    Staged set_a, set_b;
    auto fetch = [&](Staged& g_, int c0) {
        if (c0 >= n_tok) return;
#pragma unroll
        for (int r = 0; r < RK; r++) {
            const int idx = tid + r * SCAN_THREADS, t = c0 + idx / NPAD, n = idx % NPAD;
            const bool ok = t < n_tok && n < N;
            g_.k[r] = ok ? kg[(size_t)t * ldk + n] : 0.f;
            g_.q[r] = ok ? qg[(size_t)t * ldq + n] : 0.f;
            g_.a[r] = ok ? ag[(size_t)t * lda + n] : 0.f;
        }
#pragma unroll
        for (int r = 0; r < RV; r++) {
            const int idx = tid + r * SCAN_THREADS, t = c0 + idx / PT, pp = idx % PT;
            g_.v[r] = (idx < TOK * PT && t < n_tok && pz * PT + pp < P) ? vg[(size_t)t * ldv + pp] : 0.f;
        }
        g_.b = (tid < TOK && c0 + tid < n_tok) ? b[(size_t)(q0 + c0 + tid) * ldb + h] : 0.f;
    };
    auto stash = [&](const Staged& g_) {
#pragma unroll
        for (int r = 0; r < RK; r++) {
            const int idx = tid + r * SCAN_THREADS;
            k_s[idx] = g_.k[r];
            q_s[idx] = g_.q[r];
            const float z = g_.a[r] + bias_r[r];
            const float sp = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));                 // softplus, exact for every z
            g_s[idx] = expf(neg_rate * sp);
        }
#pragma unroll
        for (int r = 0; r < RV; r++)
            if (tid + r * SCAN_THREADS < TOK * PT) v_s[tid + r * SCAN_THREADS] = g_.v[r];
        if (tid < TOK) b_s[tid] = 1.0f / (1.0f + expf(-g_.b));
        __syncthreads();
        // unit vectors: a wave a token, the sums of squares in lane order then across the wave
        for (int t = wv; t < TOK; t += SCAN_THREADS / WAVE) {
            float sk = 0.f, sq = 0.f;
            for (int n = lane; n < NPAD; n += WAVE) {
                const float kv = k_s[t * NPAD + n], qv = q_s[t * NPAD + n];
                sk = fmaf(kv, kv, sk);
                sq = fmaf(qv, qv, sq);
            }
            const float ki = 1.0f / sqrtf(wave_sum(sk) + unit_eps), qi = q_scale / sqrtf(wave_sum(sq) + unit_eps);
            for (int n = lane; n < NPAD; n += WAVE) {
                k_s[t * NPAD + n] *= ki;
                q_s[t * NPAD + n] *= qi;
            }
        }
    };
    auto chunk = [&](Staged& g_, int c0) {
        const int nt = n_tok - c0 < TOK ? n_tok - c0 : TOK;
        __syncthreads();                                   // the walk before has read what is overwritten now
        stash(g_);
        __syncthreads();
        fetch(g_, c0 + 2 * TOK);
        // A token's operands leave LDS two tokens before its multiply-adds (as in linear_scan_kernel): what is left between
        // one token's state and the next is the decay, the sum over the column's lanes, the correction and the write.
        struct Operands { float4 k[NPT / 4], q[NPT / 4], g[NPT / 4]; float beta, v; };
        auto read = [&](int t, Operands& o) {
            const float4* kt = reinterpret_cast<const float4*>(k_s + t * NPAD + ns * NPT);
            const float4* qt = reinterpret_cast<const float4*>(q_s + t * NPAD + ns * NPT);
            const float4* gt = reinterpret_cast<const float4*>(g_s + t * NPAD + ns * NPT);
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                o.k[i] = kt[i];
                o.q[i] = qt[i];
                o.g[i] = gt[i];
            }
            o.beta = b_s[t];
            o.v = v_s[t * PT + pl];
        };
        auto token = [&](int t, const Operands& o) {
            float d0 = 0.f, d1 = 0.f;
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                const float4 gg = o.g[i], kk = o.k[i];
                st[4 * i] *= gg.x;
                st[4 * i + 1] *= gg.y;
                st[4 * i + 2] *= gg.z;
                st[4 * i + 3] *= gg.w;
                d0 = fmaf(st[4 * i], kk.x, d0);
                d1 = fmaf(st[4 * i + 1], kk.y, d1);
                d0 = fmaf(st[4 * i + 2], kk.z, d0);
                d1 = fmaf(st[4 * i + 3], kk.w, d1);
            }
            const float dot = run_sum<NS>(d0 + d1);
            const float u = o.beta * (o.v - dot);
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                const float4 kk = o.k[i], qq = o.q[i];
                st[4 * i] = fmaf(kk.x, u, st[4 * i]);
                st[4 * i + 1] = fmaf(kk.y, u, st[4 * i + 1]);
                st[4 * i + 2] = fmaf(kk.z, u, st[4 * i + 2]);
                st[4 * i + 3] = fmaf(kk.w, u, st[4 * i + 3]);
                acc0 = fmaf(st[4 * i], qq.x, acc0);
                acc1 = fmaf(st[4 * i + 1], qq.y, acc1);
                acc0 = fmaf(st[4 * i + 2], qq.z, acc0);
                acc1 = fmaf(st[4 * i + 3], qq.w, acc1);
            }
            part_s[t * SCAN_THREADS + tid] = acc0 + acc1;
        };
        if (AHEAD && nt == TOK) {
            Operands ring[3];
            read(0, ring[0]);
            read(1, ring[1]);
#pragma unroll
            for (int t = 0; t < TOK; t++) {
                if (t + 2 < TOK) read(t + 2, ring[(t + 2) % 3]);
                token(t, ring[t % 3]);
            }
        } else {
            for (int t = 0; t < nt; t++) {
                Operands o;
                read(t, o);
                token(t, o);
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nt * PT; idx += SCAN_THREADS) {
            const int t = idx / PT, pp = idx % PT;
            if (pz * PT + pp >= P) continue;
            const float4* sh = reinterpret_cast<const float4*>(part_s + t * SCAN_THREADS + pp * NS);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NS / 4; i++) {
                const float4 w4 = sh[i];
                acc = ((acc + w4.x) + w4.y) + w4.z + w4.w;
            }
            y[(size_t)(q0 + c0 + t) * ldy + h * P + pz * PT + pp] = acc;
        }
    };
    fetch(set_a, 0);
    fetch(set_b, TOK);
    for (int c0 = 0; c0 < n_tok; c0 += 2 * TOK) {
        chunk(set_a, c0);
        if (c0 + TOK < n_tok) chunk(set_b, c0 + TOK);
    }
#pragma unroll
    for (int i = 0; i < NPT; i++) S[(size_t)i * p_pad * NS] = st[i];
}

extern "C" int hfa_delta_scan(const float* q, int ldq, const float* k, int ldk, int qk_heads, int qk_dim, const float* v, int ldv,
                              int n_heads, int v_dim, const float* a, int lda, const float* dt_bias, const float* a_log,
                              const float* b, int ldb, float q_scale, float unit_eps, float* state, size_t state_ld,
                              const int* q_start, const int* seq_slot, int n_seqs, int max_q_len, float* y, int ldy, hipStream_t stream) {
    HFA_REQUIRE(q && k && v && a && dt_bias && a_log && b && state && q_start && seq_slot && y && n_seqs > 0, "delta_scan: a null argument");
    HFA_REQUIRE(n_heads > 0 && qk_heads > 0 && n_heads % qk_heads == 0 && qk_dim > 0 && v_dim > 0,
                "delta_scan: %d heads over %d heads of keys", n_heads, qk_heads);
    HFA_REQUIRE(qk_dim <= 256, "delta_scan: a state of %d rows a head is too large (at most 256)", qk_dim);
    HFA_REQUIRE(ldq >= qk_heads * qk_dim && ldk >= qk_heads * qk_dim && ldv >= n_heads * v_dim && ldy >= n_heads * v_dim &&
                    lda >= n_heads * qk_dim && ldb >= n_heads && state_ld >= hfa_linear_scan_state_floats(n_heads, qk_dim, v_dim),
                "delta_scan: a row is shorter than its heads (a state row holds hfa_linear_scan_state_floats values)");
    int ns, npt;
    scan_shape(qk_dim, &ns, &npt);
    const int pt = SCAN_THREADS / ns, p_tiles = (v_dim + pt - 1) / pt;
    HFA_REQUIRE(n_heads <= 65535 && n_seqs <= 65535 && p_tiles <= 65535, "delta_scan: the step exceeds the grid");
    dim3 grid(n_heads, n_seqs, p_tiles);
    const bool ahead = max_q_len >= SCAN_TOKENS;            // some request brings a whole chunk
#define DELTA_ARGS q, ldq, k, ldk, n_heads / qk_heads, qk_dim, v, ldv, v_dim, a, lda, dt_bias, a_log, b, ldb, q_scale, unit_eps, state, state_ld, q_start, seq_slot, y, ldy
#define DELTA_GO(NS, NPT)                                                                              \
    do {                                                                                               \
        if (ahead) delta_scan_kernel<NS, NPT, true><<<grid, SCAN_THREADS, 0, stream>>>(DELTA_ARGS);   \
        else delta_scan_kernel<NS, NPT, false><<<grid, SCAN_THREADS, 0, stream>>>(DELTA_ARGS);        \
    } while (0)
    if (ns == 4) DELTA_GO(4, 4);
    else if (ns == 8 && npt == 4) DELTA_GO(8, 4);
    else if (ns == 8) DELTA_GO(8, 8);
    else if (npt == 4) DELTA_GO(16, 4);
    else if (npt == 8) DELTA_GO(16, 8);
    else DELTA_GO(16, 16);
#undef DELTA_GO
#undef DELTA_ARGS
    HFA_LAUNCH_CHECK("delta_scan");
    return 0;
}

// ---- a decay per key channel -------------------------------------------------------------------------------------------
// Per head, S [N][P] in the state row, in hfa_linear_scan's layout: S <- diag(a_t) S + k_t v_t^T, y_t = S^T (q_scale q_t), with
// the decays a_t[n] given in fp32 ([T, H N], formed beforehand by hfa_channel_decay: every block of a head's columns would
// otherwise form the same decays again). kcomp 1: the key is the decay's complement, k = 1 - a (a forget gate that also decides
// what is written; no keys are read); else keys are read. q_act HFA_ACT_SILU: the queries pass silu on their way in. The block,
// its lanes and the staging through LDS are linear_scan_kernel's, with the decays staged beside the keys as delta_scan_kernel
// stages its own; nothing crosses lanes inside the walk.
template <typename T, int NS, int NPT>
__global__ __launch_bounds__(SCAN_THREADS) void channel_scan_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, int N, const T* __restrict__ v, int ldv, int P,
    const float* __restrict__ decay, int ld_decay, int kcomp, int q_act, float q_scale, float* __restrict__ state, size_t state_ld, const int* __restrict__ q_start,
    const int* __restrict__ seq_slot, float* __restrict__ y, int ldy) {
    constexpr int NPAD = NS * NPT, PT = SCAN_THREADS / NS, TOK = SCAN_TOKENS;
    constexpr int RK = TOK * NPAD / SCAN_THREADS, RV = (TOK * PT + SCAN_THREADS - 1) / SCAN_THREADS;
    static_assert(TOK * NPAD % SCAN_THREADS == 0 && NPT % 4 == 0, "the staging loops are whole");
    __shared__ __attribute__((aligned(16))) float k_s[TOK * NPAD];
    __shared__ __attribute__((aligned(16))) float q_s[TOK * NPAD];
    __shared__ __attribute__((aligned(16))) float g_s[TOK * NPAD];
    __shared__ float v_s[TOK * PT];
    __shared__ __attribute__((aligned(16))) float part_s[TOK * SCAN_THREADS];
    const int h = blockIdx.x, s = blockIdx.y, pz = blockIdx.z, tid = threadIdx.x;
    const int pl = tid / NS, ns = tid % NS;
    const int q0 = q_start[s], n_tok = q_start[s + 1] - q0;
    if (n_tok <= 0) return;
    const int p_pad = (int)gridDim.z * PT;
    float* S = state + (size_t)seq_slot[s] * state_ld + (size_t)h * NPT * p_pad * NS + (size_t)pz * SCAN_THREADS + tid;
    float st[NPT];
#pragma unroll
    for (int i = 0; i < NPT; i++) st[i] = S[(size_t)i * p_pad * NS];
    const T* kg = k ? k + (size_t)q0 * ldk + h * N : nullptr;
    const T* qg = q + (size_t)q0 * ldq + h * N;
    const float* gg = decay + (size_t)q0 * ld_decay + h * N;
    const T* vg = v + (size_t)q0 * ldv + h * P + pz * PT;
    struct Staged { float k[RK], q[RK], z[RK], v[RV]; };
    Staged set_a, set_b;
    auto fetch = [&](Staged& g_, int c0) {
        if (c0 >= n_tok) return;
#pragma unroll
        for (int r = 0; r < RK; r++) {
            const int idx = tid + r * SCAN_THREADS, t = c0 + idx / NPAD, n = idx % NPAD;
            const bool ok = t < n_tok && n < N;
            g_.k[r] = (ok && !kcomp) ? to_f32(kg[(size_t)t * ldk + n]) : 0.f;
            g_.q[r] = ok ? to_f32(qg[(size_t)t * ldq + n]) : 0.f;
            g_.z[r] = ok ? gg[(size_t)t * ld_decay + n] : 0.f;
        }
#pragma unroll
        for (int r = 0; r < RV; r++) {
            const int idx = tid + r * SCAN_THREADS, t = c0 + idx / PT, pp = idx % PT;
            g_.v[r] = (idx < TOK * PT && t < n_tok && pz * PT + pp < P) ? to_f32(vg[(size_t)t * ldv + pp]) : 0.f;
        }
    };
    auto stash = [&](const Staged& g_) {
#pragma unroll
        for (int r = 0; r < RK; r++) {
            const int idx = tid + r * SCAN_THREADS, n = idx % NPAD;
            const float a = g_.z[r], kk = kcomp ? 1.0f - a : g_.k[r];
            const bool live = n < N;                       // rows beyond N stay zero
            g_s[idx] = live ? a : 0.f;
            k_s[idx] = live ? kk : 0.f;
            const float qv = g_.q[r];
            q_s[idx] = (q_act == HFA_ACT_SILU ? qv / (1.0f + expf(-qv)) : qv) * q_scale;
        }
#pragma unroll
        for (int r = 0; r < RV; r++)
            if (tid + r * SCAN_THREADS < TOK * PT) v_s[tid + r * SCAN_THREADS] = g_.v[r];
    };
    auto chunk = [&](Staged& g_, int c0) {
        const int nt = n_tok - c0 < TOK ? n_tok - c0 : TOK;
        __syncthreads();                                   // the walk before has read what is overwritten now
        stash(g_);
        __syncthreads();
        fetch(g_, c0 + 2 * TOK);
        struct Operands { float4 k[NPT / 4], q[NPT / 4], g[NPT / 4]; float v; };
        auto read = [&](int t, Operands& o) {
            const float4* kt = reinterpret_cast<const float4*>(k_s + t * NPAD + ns * NPT);
            const float4* qt = reinterpret_cast<const float4*>(q_s + t * NPAD + ns * NPT);
            const float4* gt = reinterpret_cast<const float4*>(g_s + t * NPAD + ns * NPT);
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                o.k[i] = kt[i];
                o.q[i] = qt[i];
                o.g[i] = gt[i];
            }
            o.v = v_s[t * PT + pl];
        };
        auto token = [&](int t, const Operands& o) {
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int i = 0; i < NPT / 4; i++) {
                const float4 a4 = o.g[i], kk = o.k[i], qq = o.q[i];
                st[4 * i] = fmaf(a4.x, st[4 * i], kk.x * o.v);
                st[4 * i + 1] = fmaf(a4.y, st[4 * i + 1], kk.y * o.v);
                st[4 * i + 2] = fmaf(a4.z, st[4 * i + 2], kk.z * o.v);
                st[4 * i + 3] = fmaf(a4.w, st[4 * i + 3], kk.w * o.v);
                acc0 = fmaf(st[4 * i], qq.x, acc0);
                acc1 = fmaf(st[4 * i + 1], qq.y, acc1);
                acc0 = fmaf(st[4 * i + 2], qq.z, acc0);
                acc1 = fmaf(st[4 * i + 3], qq.w, acc1);
            }
            part_s[t * SCAN_THREADS + tid] = acc0 + acc1;
        };
        if (nt == TOK) {
            Operands ring[3];
            read(0, ring[0]);
            read(1, ring[1]);
#pragma unroll
            for (int t = 0; t < TOK; t++) {
                if (t + 2 < TOK) read(t + 2, ring[(t + 2) % 3]);
                token(t, ring[t % 3]);
            }
        } else {
            for (int t = 0; t < nt; t++) {
                Operands o;
                read(t, o);
                token(t, o);
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nt * PT; idx += SCAN_THREADS) {
            const int t = idx / PT, pp = idx % PT;
            if (pz * PT + pp >= P) continue;
            const float4* sh = reinterpret_cast<const float4*>(part_s + t * SCAN_THREADS + pp * NS);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NS / 4; i++) {
                const float4 w4 = sh[i];
                acc = ((acc + w4.x) + w4.y) + w4.z + w4.w;
            }
            y[(size_t)(q0 + c0 + t) * ldy + h * P + pz * PT + pp] = acc;
        }
    };
    fetch(set_a, 0);
    fetch(set_b, TOK);
    for (int c0 = 0; c0 < n_tok; c0 += 2 * TOK) {
        chunk(set_a, c0);
        if (c0 + TOK < n_tok) chunk(set_b, c0 + TOK);
    }
#pragma unroll
    for (int i = 0; i < NPT; i++) S[(size_t)i * p_pad * NS] = st[i];
}

// The decays of hfa_channel_scan, in fp32, from x = z[r, c] + bias[c] (bias null: 0):
//   form 0: a = lower[c] + (1 - lower[c]) sigmoid(x)                                 (a forget gate with a lower bound)
//   form 1: a = sigmoid(x)^inv_tau, as exp(inv_tau logsigmoid(x))                    (a root of a sigmoid)
template <typename TG>
__global__ void channel_decay_kernel(const TG* __restrict__ z, int ldz, const float* __restrict__ bias, int form, const float* __restrict__ lower,
                                     float inv_tau, float* __restrict__ out, int ldo, int width, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / width, c = i % width;
        const float x = to_f32(z[r * ldz + c]) + (bias ? bias[c] : 0.f);
        float a;
        if (form == 0) {
            const float lo = lower[c];
            a = lo + (1.0f - lo) * (1.0f / (1.0f + expf(-x)));
        } else {
            const float ls = -(fmaxf(-x, 0.f) + log1pf(expf(-fabsf(x))));       // logsigmoid, exact for every x
            a = expf(inv_tau * ls);
        }
        out[r * ldo + c] = a;
    }
}

extern "C" int hfa_channel_decay(const void* z, int z_dtype, int ldz, const float* bias, int form, const float* lower, float inv_tau,
                                 float* out, int ldo, int n_rows, int width, hipStream_t stream) {
    HFA_REQUIRE(z && out && n_rows > 0 && width > 0 && ldz >= width && ldo >= width, "channel_decay: bad arguments");
    HFA_REQUIRE((form == 0 && lower) || (form == 1 && inv_tau > 0.f), "channel_decay: form 0 needs lower bounds, form 1 a positive 1 / tau");
    HFA_REQUIRE(z_dtype == HFA_F32 || z_dtype == HFA_BF16, "channel_decay: unknown dtype %d", z_dtype);
    const size_t total = (size_t)n_rows * width;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (z_dtype == HFA_F32) channel_decay_kernel<float><<<blocks, 256, 0, stream>>>((const float*)z, ldz, bias, form, lower, inv_tau, out, ldo, width, total);
    else channel_decay_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)z, ldz, bias, form, lower, inv_tau, out, ldo, width, total);
    HFA_LAUNCH_CHECK("channel_decay");
    return 0;
}

extern "C" int hfa_channel_scan(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype, const float* decay,
                                int ld_decay, int kcomp, int q_act, int n_heads, int qk_dim, int v_dim, float q_scale, float* state,
                                size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs, float* y, int ldy, hipStream_t stream) {
    HFA_REQUIRE(q && v && decay && state && q_start && seq_slot && y && n_seqs > 0 && (kcomp || k), "channel_scan: a null argument");
    HFA_REQUIRE(n_heads > 0 && qk_dim > 0 && v_dim > 0, "channel_scan: bad sizes");
    HFA_REQUIRE(q_act == HFA_ACT_NONE || q_act == HFA_ACT_SILU, "channel_scan: the queries pass silu or nothing");
    HFA_REQUIRE(qk_dim <= 256, "channel_scan: a state of %d rows a head is too large (at most 256)", qk_dim);
    HFA_REQUIRE(ldq >= n_heads * qk_dim && (kcomp || ldk >= n_heads * qk_dim) && ldv >= n_heads * v_dim && ldy >= n_heads * v_dim &&
                    ld_decay >= n_heads * qk_dim && state_ld >= hfa_linear_scan_state_floats(n_heads, qk_dim, v_dim),
                "channel_scan: a row is shorter than its heads (a state row holds hfa_linear_scan_state_floats values)");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "channel_scan: unknown dtype %d", dtype);
    int ns, npt;
    scan_shape(qk_dim, &ns, &npt);
    const int pt = SCAN_THREADS / ns, p_tiles = (v_dim + pt - 1) / pt;
    HFA_REQUIRE(n_heads <= 65535 && n_seqs <= 65535 && p_tiles <= 65535, "channel_scan: the step exceeds the grid");
    dim3 grid(n_heads, n_seqs, p_tiles);
#define CH_GO(T, NS, NPT)                                                                                                      \
    channel_scan_kernel<T, NS, NPT><<<grid, SCAN_THREADS, 0, stream>>>((const T*)q, ldq, (const T*)k, ldk, qk_dim, (const T*)v, ldv, v_dim, \
                                                                       decay, ld_decay, kcomp, q_act, q_scale, state, state_ld, q_start,  \
                                                                       seq_slot, y, ldy)
#define CH_SIZES(T)                                          \
    do {                                                     \
        if (ns == 4) CH_GO(T, 4, 4);                         \
        else if (ns == 8 && npt == 4) CH_GO(T, 8, 4);        \
        else if (ns == 8) CH_GO(T, 8, 8);                    \
        else if (npt == 4) CH_GO(T, 16, 4);                  \
        else if (npt == 8) CH_GO(T, 16, 8);                  \
        else CH_GO(T, 16, 16);                               \
    } while (0)
    if (dtype == HFA_F32) CH_SIZES(float);
    else CH_SIZES(bf16);
#undef CH_SIZES
#undef CH_GO
    HFA_LAUNCH_CHECK("channel_scan");
    return 0;
}
