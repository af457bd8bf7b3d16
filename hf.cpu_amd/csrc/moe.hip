// Mixture of experts: the router's choice, the plan of a step (which rows go to which expert), the products of all
// experts in one launch, and the weighted sum into the residual stream.
//
//   hfa_moe_route    fp32 router logits -> the chosen experts of each token and their weights
//   hfa_moe_plan     the (token, choice) pairs put in the order of their experts, and the tiles of rows that the
//                    products walk: nothing of a step's routing is known to the host
//   hfa_moe_gemm     out[row] = act(a[src(row)] . w[expert of row]^T), one block a tile of rows of one expert
//   hfa_moe_combine  x[t] += sum over the token's choices, in the order of the choices
//
// A row's result depends on its own operands only and is summed over K in one fixed order, so neither the rest of the
// batch nor the place that a pair got inside its expert's run changes it.
#include "api.h"
#include "common.h"

#define MOE_MAX_EXPERTS 1024

// ---- router -----------------------------------------------------------------------------
// The better of two candidates: the larger score, the lower index among equals.
__device__ __forceinline__ void better(float& v, int& i, float v2, int i2) {
    if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
}
__device__ __forceinline__ void wave_best(float& v, int& i) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        const float v2 = __shfl_xor(v, off, WAVE);
        const int i2 = __shfl_xor(i, off, WAVE);
        better(v, i, v2, i2);
    }
}

// One wave a token. score = softmax over all experts (or the logistic function of each logit, `scoring` 1; or, `scoring` 2,
// exp(logit - the largest logit), which with `renorm` makes the weights the softmax over the chosen logits alone); experts
// form n_groups runs of neighbours, a run scores as its best expert, and only experts of the `keep` best runs can
// be chosen; the `top` best of those are chosen, and weigh score / (sum of the chosen scores + 1e-20) if `renorm`,
// else their score; times `out_scale`.
__global__ __launch_bounds__(WAVE) void moe_route_kernel(const float* __restrict__ logits, int ld, int E, int top,
                                                        int n_groups, int keep, int scoring, int renorm, float out_scale,
                                                        int* __restrict__ ids, float* __restrict__ weights) {
    __shared__ float s[MOE_MAX_EXPERTS];
    __shared__ float gs[MOE_MAX_EXPERTS];
    __shared__ unsigned char open_s[MOE_MAX_EXPERTS];        // per group: may be chosen from
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * ld;
    if (scoring == 0) {
        float m = -INFINITY;
        for (int e = lane; e < E; e += WAVE) m = fmaxf(m, z[e]);
        m = wave_max(m);
        float sum = 0.f;
        for (int e = lane; e < E; e += WAVE) {
            const float p = expf(z[e] - m);
            s[e] = p;
            sum += p;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += WAVE) s[e] = s[e] / sum;
    } else if (scoring == 2) {
        float m = -INFINITY;
        for (int e = lane; e < E; e += WAVE) m = fmaxf(m, z[e]);
        m = wave_max(m);
        for (int e = lane; e < E; e += WAVE) s[e] = expf(z[e] - m);
    } else {
        for (int e = lane; e < E; e += WAVE) s[e] = 1.0f / (1.0f + expf(-z[e]));
    }
    __syncthreads();
    const int per = E / n_groups;
    for (int g = lane; g < n_groups; g += WAVE) {
        float b = -INFINITY;
        for (int e = g * per; e < (g + 1) * per; e++) b = fmaxf(b, s[e]);
        gs[g] = b;
        open_s[g] = keep >= n_groups ? 1 : 0;
    }
    __syncthreads();
    if (keep < n_groups) {
        for (int r = 0; r < keep; r++) {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int g = lane; g < n_groups; g += WAVE)
                if (!open_s[g]) better(bv, bi, gs[g], g);
            wave_best(bv, bi);
            if (lane == 0 && bi < n_groups) open_s[bi] = 1;
            __syncthreads();
        }
    }
    float chosen_sum = 0.f;
    for (int r = 0; r < top; r++) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int e = lane; e < E; e += WAVE)
            if (open_s[e / per] && s[e] >= 0.f) better(bv, bi, s[e], e);
        wave_best(bv, bi);
        if (bi >= E) { bi = 0; bv = 0.f; }                   // fewer open experts than choices: weight nothing
        else if (lane == 0) s[bi] = -1.f;                    // taken
        if (lane == 0) {
            ids[(size_t)t * top + r] = bi;
            weights[(size_t)t * top + r] = bv;
        }
        chosen_sum += bv;
        __syncthreads();
    }
    if (lane < top) {
        const float wv = weights[(size_t)t * top + lane];
        weights[(size_t)t * top + lane] = (renorm ? wv / (chosen_sum + 1e-20f) : wv) * out_scale;
    }
}

extern "C" int hfa_moe_route(const float* logits, int ld, int n_tokens, int n_experts, int top, int n_groups, int keep,
                             int scoring, int renorm, float out_scale, int* ids, float* weights, hipStream_t stream) {
    HFA_REQUIRE(logits && ids && weights && n_tokens > 0, "moe_route: bad arguments");
    HFA_REQUIRE(n_experts > 0 && n_experts <= MOE_MAX_EXPERTS && ld >= n_experts, "moe_route: %d experts (at most %d)", n_experts,
                MOE_MAX_EXPERTS);
    HFA_REQUIRE(top > 0 && top <= WAVE && top <= n_experts, "moe_route: %d choices of %d experts (at most %d)", top, n_experts, WAVE);
    HFA_REQUIRE(n_groups > 0 && n_experts % n_groups == 0 && keep > 0 && keep <= n_groups,
                "moe_route: %d experts do not form %d equal groups of which %d are kept", n_experts, n_groups, keep);
    HFA_REQUIRE(scoring >= 0 && scoring <= 2, "moe_route: unknown scoring %d", scoring);
    moe_route_kernel<<<n_tokens, WAVE, 0, stream>>>(logits, ld, n_experts, top, n_groups, keep, scoring, renorm, out_scale, ids,
                                                    weights);
    HFA_LAUNCH_CHECK("moe_route");
    return 0;
}

// ---- plan -------------------------------------------------------------------------------
// Pair p = token * top + choice goes to expert ids[p]. row_pair[r] = the pair in row r of the expert-ordered rows;
// tiles[3 i ..] = (expert, first row, rows) of tile i, tiles of at most tile_rows rows of one expert; *n_tiles their
// number (at most n_pairs / tile_rows + n_experts). One block.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int n_pairs, int E, int tile_rows,
                                                       int* __restrict__ row_pair, int* __restrict__ tiles,
                                                       int* __restrict__ n_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS];
    __shared__ int start[MOE_MAX_EXPERTS];
    __shared__ int tile0[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&count[ids[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int rows = 0, nt = 0;
        for (int e = 0; e < E; e++) {
            start[e] = rows;
            tile0[e] = nt;
            rows += count[e];
            nt += (count[e] + tile_rows - 1) / tile_rows;
        }
        *n_tiles = nt;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int c = count[e];
        for (int i = 0, r = 0; r < c; i++, r += tile_rows) {
            int* tl = tiles + 3 * (tile0[e] + i);
            tl[0] = e;
            tl[1] = start[e] + r;
            tl[2] = c - r < tile_rows ? c - r : tile_rows;
        }
    }
    __syncthreads();
    // Where a pair lands inside its expert's run is whatever order the atomics give: a row's result does not depend
    // on its place (see the head of this file).
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) row_pair[atomicAdd(&start[ids[p]], 1)] = p;
}

extern "C" int hfa_moe_plan(const int* ids, int n_pairs, int n_experts, int tile_rows, int* row_pair, int* tiles,
                            int* n_tiles, hipStream_t stream) {
    HFA_REQUIRE(ids && row_pair && tiles && n_tiles && n_pairs > 0 && tile_rows > 0, "moe_plan: bad arguments");
    HFA_REQUIRE(n_experts > 0 && n_experts <= MOE_MAX_EXPERTS, "moe_plan: %d experts (at most %d)", n_experts, MOE_MAX_EXPERTS);
    int threads = n_pairs >= 1024 ? 1024 : (n_pairs + WAVE - 1) / WAVE * WAVE;
    moe_plan_kernel<<<1, threads, 0, stream>>>(ids, n_pairs, n_experts, tile_rows, row_pair, tiles, n_tiles);
    HFA_LAUNCH_CHECK("moe_plan");
    return 0;
}

// ---- the experts' products ----------------------------------------------------------------
// Gated experts (`gated` in the kernels below): the rows of an expert's matrix come in blocks of 32 gate rows, 32 up rows,
// and a product's last lines form, from the two 32-bit sums of a pair of such blocks, g sigmoid(alpha g) (u + shift) with
// g = min(c gate, limit), u = clamp(c up, -limit, limit) (limit <= 0: unbounded), c the row's pair_scale (null: 1):
// scaling the sums is scaling the expert's input. The output then has N / 2 columns.
struct GatedAct { float alpha, limit, shift; };
__device__ __forceinline__ float gated_apply(float g, float u, float c, const GatedAct ga) {
    g *= c;
    u *= c;
    if (ga.limit > 0.f) {
        g = fminf(g, ga.limit);
        u = fminf(fmaxf(u, -ga.limit), ga.limit);
    }
    return g / (1.0f + expf(-ga.alpha * g)) * (u + ga.shift);
}

// Plain form, any dtype and shape: a tile of up to 32 rows x 64 columns a block, operands staged through LDS 32 k at a
// time, every output summed over k in ascending order by one thread.
#define PM 32
#define PN 64
#define PK 32
template <typename T, typename TW, typename TO>
__global__ __launch_bounds__(256) void moe_gemm_plain_kernel(
    const T* __restrict__ a, int lda, int a_div, const TW* __restrict__ w, const int* __restrict__ row_pair,
    const int* __restrict__ tiles, const int* __restrict__ n_tiles, TO* __restrict__ out, int ldo, int out_by_pair,
    const float* __restrict__ pair_scale, int act, int N, int K, int gated, GatedAct ga) {
    if ((int)blockIdx.x >= *n_tiles) return;
    __shared__ float a_s[PM][PK + 1];
    __shared__ float w_s[PN][PK + 1];
    __shared__ float o_s[PM][PN + 1];
    __shared__ int src_s[PM], pair_s[PM];
    const int e = tiles[3 * blockIdx.x], r0 = tiles[3 * blockIdx.x + 1], nr = tiles[3 * blockIdx.x + 2];
    const int n0 = blockIdx.y * PN, tid = threadIdx.x;
    if (tid < PM) {
        const int pair = row_pair[r0 + (tid < nr ? tid : 0)];
        pair_s[tid] = pair;
        src_s[tid] = a_div > 0 ? pair / a_div : r0 + (tid < nr ? tid : 0);
    }
    __syncthreads();
    const TW* we = w + (size_t)e * N * K;
    const int col = tid & (PN - 1), rg = tid / PN;          // 4 row groups of 8 rows
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;
    for (int k0 = 0; k0 < K; k0 += PK) {
        for (int i = tid; i < PM * PK; i += 256) {
            const int r = i / PK, k = i % PK;
            a_s[r][k] = k0 + k < K ? to_f32(a[(size_t)src_s[r] * lda + k0 + k]) : 0.f;
        }
        for (int i = tid; i < PN * PK; i += 256) {
            const int n = i / PK, k = i % PK;
            w_s[n][k] = (k0 + k < K && n0 + n < N) ? to_f32(we[(size_t)(n0 + n) * K + k0 + k]) : 0.f;
        }
        __syncthreads();
        const int kn = K - k0 < PK ? K - k0 : PK;
        for (int k = 0; k < kn; k++) {
            const float wv = w_s[col][k];
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = fmaf(a_s[rg * 8 + i][k], wv, acc[i]);
        }
        __syncthreads();
    }
    if (gated) {                                            // columns c and c + 32 of the tile are gate and up of one output
#pragma unroll
        for (int i = 0; i < 8; i++) o_s[rg * 8 + i][col] = acc[i];
        __syncthreads();
        for (int i = tid; i < PM * (PN / 2); i += 256) {
            const int r = i / (PN / 2), c = i % (PN / 2);
            if (r >= nr || n0 + 32 + c >= N) continue;
            const float sc = pair_scale ? pair_scale[pair_s[r]] : 1.f;
            const size_t orow = out_by_pair ? (size_t)pair_s[r] : (size_t)(r0 + r);
            out[orow * ldo + n0 / 2 + c] = from_f32<TO>(gated_apply(o_s[r][c], o_s[r][c + 32], sc, ga));
        }
        return;
    }
    if (n0 + col >= N) return;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int r = rg * 8 + i;
        if (r >= nr) continue;
        float v = hfa_act_apply(act, acc[i]);
        if (pair_scale) v *= pair_scale[pair_s[r]];
        const size_t orow = out_by_pair ? (size_t)pair_s[r] : (size_t)(r0 + r);
        out[orow * ldo + n0 + col] = from_f32<TO>(v);
    }
}

// Matrix-core form (bf16 operands, K a multiple of 16, N of 32): a block of four waves owns 32 RM rows x 128 CN columns
// of one expert, a wave 32 RM x 32 CN of them. Both operands are K-contiguous, so a lane's 8 consecutive k of one row
// are one 16-byte load straight into the operand registers of v_mfma_f32_32x32x16_bf16; the four waves of a block read
// the same rows of `a`, which the CU's cache serves after the first.
typedef __bf16 mbf16x8 __attribute__((ext_vector_type(8)));
typedef float mfloatx16 __attribute__((ext_vector_type(16)));
union MFrag {
    uint4 u;
    mbf16x8 v;
};

// Few rows an expert (decoded tokens): the experts' matrices are streamed once and that stream is the bound, so the
// work is cut small: a block owns 32 rows x 32 columns of one expert, its four waves take a quarter of K each (K a
// multiple of 64) with the loads of four steps on their way at a time, and the four partial tiles are added in LDS in
// wave order.
template <typename TO, bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_split_kernel(
    const uint16_t* __restrict__ a, int lda, int a_div, const uint16_t* __restrict__ w, const int* __restrict__ row_pair,
    const int* __restrict__ tiles, const int* __restrict__ n_tiles, TO* __restrict__ out, int ldo, int out_by_pair,
    const float* __restrict__ pair_scale, int act, int N, int K, GatedAct ga) {
    if ((int)blockIdx.x >= *n_tiles) return;
    constexpr int NB = GATED ? 2 : 1;                       // gated: a block owns a block of 32 gate rows and its 32 up rows
    __shared__ float part_s[4][NB][32 * 33];
    const int e = tiles[3 * blockIdx.x], r0 = tiles[3 * blockIdx.x + 1], nr = tiles[3 * blockIdx.x + 2];
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1), col = lane & 31, half = lane >> 5;
    const int n0 = blockIdx.y * 32 * NB;
    const int row = r0 + (col < nr ? col : 0);
    const int src = a_div > 0 ? row_pair[row] / a_div : row;
    const int kq = K / 4, k0 = wave * kq;
    const uint16_t* ap = a + (size_t)src * lda + k0 + half * 8;
    const uint16_t* wp[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) {
        int n = n0 + 32 * b + col;
        n = n < N ? n : N - 1;
        wp[b] = w + ((size_t)e * N + n) * K + k0 + half * 8;
    }
    mfloatx16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = 0.f;
    int k = 0;
    for (; k + 64 <= kq; k += 64) {
        MFrag af[4], wf[NB][4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int b = 0; b < NB; b++) wf[b][u].u = *reinterpret_cast<const uint4*>(wp[b] + k + 16 * u);
            af[u].u = *reinterpret_cast<const uint4*>(ap + k + 16 * u);
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int b = 0; b < NB; b++) acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[u].v, wf[b][u].v, acc[b], 0, 0, 0);
    }
    for (; k < kq; k += 16) {
        MFrag af, wf;
        af.u = *reinterpret_cast<const uint4*>(ap + k);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            wf.u = *reinterpret_cast<const uint4*>(wp[b] + k);
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af.v, wf.v, acc[b], 0, 0, 0);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) part_s[wave][b][(8 * (r / 4) + 4 * half + (r % 4)) * 33 + col] = acc[b][r];
    __syncthreads();
    for (int i = threadIdx.x; i < 32 * 32; i += 256) {
        const int r = i >> 5, c = i & 31;
        if (r >= nr || n0 + 32 * (NB - 1) + c >= N) continue;
        float v[NB];
#pragma unroll
        for (int b = 0; b < NB; b++)
            v[b] = ((part_s[0][b][r * 33 + c] + part_s[1][b][r * 33 + c]) + part_s[2][b][r * 33 + c]) + part_s[3][b][r * 33 + c];
        const int pair = (out_by_pair || pair_scale) ? row_pair[r0 + r] : 0;
        const size_t orow = out_by_pair ? (size_t)pair : (size_t)(r0 + r);
        const float sc = pair_scale ? pair_scale[pair] : 1.f;
        if (GATED) out[orow * ldo + n0 / 2 + c] = from_f32<TO>(gated_apply(v[0], v[NB - 1], sc, ga));
        else out[orow * ldo + n0 + c] = from_f32<TO>(hfa_act_apply(act, v[0]) * sc);
    }
}

template <int RM, int CN, typename TO>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(
    const uint16_t* __restrict__ a, int lda, int a_div, const uint16_t* __restrict__ w, const int* __restrict__ row_pair,
    const int* __restrict__ tiles, const int* __restrict__ n_tiles, TO* __restrict__ out, int ldo, int out_by_pair,
    const float* __restrict__ pair_scale, int act, int N, int K, int gated, GatedAct ga) {
    if ((int)blockIdx.x >= *n_tiles) return;
    const int e = tiles[3 * blockIdx.x], r0 = tiles[3 * blockIdx.x + 1], nr = tiles[3 * blockIdx.x + 2];
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1), col = lane & 31, half = lane >> 5;
    const int n0 = (blockIdx.y * 4 + wave) * 32 * CN;
    if (n0 >= N) return;
    const uint16_t* ap[RM];
#pragma unroll
    for (int i = 0; i < RM; i++) {
        const int r = 32 * i + col;
        const int row = r0 + (r < nr ? r : 0);
        const int src = a_div > 0 ? row_pair[row] / a_div : row;
        ap[i] = a + (size_t)src * lda + half * 8;
    }
    const uint16_t* wp[CN];
#pragma unroll
    for (int j = 0; j < CN; j++) {
        int n = n0 + 32 * j + col;
        n = n < N ? n : N - 1;
        wp[j] = w + ((size_t)e * N + n) * K + half * 8;
    }
    mfloatx16 acc[RM][CN];
#pragma unroll
    for (int i = 0; i < RM; i++)
#pragma unroll
        for (int j = 0; j < CN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
#pragma unroll 2
    for (int k = 0; k < K; k += 16) {
        MFrag af[RM], wf[CN];
#pragma unroll
        for (int i = 0; i < RM; i++) af[i].u = *reinterpret_cast<const uint4*>(ap[i] + k);
#pragma unroll
        for (int j = 0; j < CN; j++) wf[j].u = *reinterpret_cast<const uint4*>(wp[j] + k);
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int j = 0; j < CN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i].v, wf[j].v, acc[i][j], 0, 0, 0);
    }
    // element r of a lane: row 8 (r / 4) + 4 half + r % 4, column lane % 32 of its 32 x 32 block
#pragma unroll
    for (int i = 0; i < RM; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = 32 * i + 8 * (r / 4) + 4 * half + (r % 4);
            if (row >= nr) continue;
            const int pair = (out_by_pair || pair_scale) ? row_pair[r0 + row] : 0;
            const float sc = pair_scale ? pair_scale[pair] : 1.f;
            const size_t orow = out_by_pair ? (size_t)pair : (size_t)(r0 + row);
            if (gated) {                                    // (CN is 2: a wave's two blocks of 32 columns are gate and up)
                if (n0 + 32 * (CN - 1) + col < N)
                    out[orow * ldo + n0 / 2 + col] = from_f32<TO>(gated_apply(acc[i][0][r], acc[i][CN - 1][r], sc, ga));
                continue;
            }
#pragma unroll
            for (int j = 0; j < CN; j++) {
                const int n = n0 + 32 * j + col;
                if (n < N) out[orow * ldo + n] = from_f32<TO>(hfa_act_apply(act, acc[i][j][r]) * sc);
            }
        }
    }
}

// Matrix-core form for many rows an expert (prompt portions): a block of WM x WN waves owns BM rows of one expert x BN
// columns and walks K in steps of BK through two LDS stages, as gemm_mfma_kernel does for one matrix: the next tile
// travels global -> registers while the current one is multiplied out of LDS, then registers -> LDS, one barrier a
// step; LDS rows are padded by 8 elements so that the 16-byte fragment reads do not conflict. The rows of `a` are
// gathered through row_pair (their source rows wait in LDS), so every operand element is read from memory once a
// block instead of once a wave.
template <int BM, int BN, int BK, int WM, int WN, typename TO>
__global__ __launch_bounds__(WM * WN * WAVE) void moe_gemm_lds_kernel(
    const uint16_t* __restrict__ a, int lda, int a_div, const uint16_t* __restrict__ w, const int* __restrict__ row_pair,
    const int* __restrict__ tiles, const int* __restrict__ n_tiles, TO* __restrict__ out, int ldo, int out_by_pair,
    const float* __restrict__ pair_scale, int act, int N, int K, int n_col_tiles, int gated, GatedAct ga) {
    constexpr int STRIDE = BK + 8, NT = WM * WN * WAVE, CPR = BK / 8, A_CH = BM * CPR / NT, W_CH = BN * CPR / NT;
    constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32, STAGE = (BM + BN) * STRIDE;
    static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0 && TM % 32 == 0 && TN % 32 == 0, "tiles spread evenly");
    // Which (tile of rows, tile of columns): block ids are dealt round-robin to the 8 XCDs, each with an L2 of its own.
    // The units, in the order (tile of rows, tile of columns), are cut into eight contiguous runs, one an XCD: the
    // blocks that share a tile's rows, and the tiles that share an expert's matrix, then meet in one L2.
    const int n_units = *n_tiles * n_col_tiles, per_xcd = (n_units + 7) / 8;
    const int unit = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || unit >= n_units) return;
    const int tile = unit / n_col_tiles;
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];       // two stages of (BM + BN) x STRIDE elements
    __shared__ int src_s[BM], pair_s[BM];
    const int e = tiles[3 * tile], r0 = tiles[3 * tile + 1], nr = tiles[3 * tile + 2];
    const int n0 = (unit % n_col_tiles) * BN, tid = threadIdx.x, wave = tid / WAVE, lane = tid & (WAVE - 1);
    const int wm = wave / WN, wn = wave % WN;
    for (int i = tid; i < BM; i += NT) {
        const int row = r0 + (i < nr ? i : 0);
        const int pair = row_pair[row];
        pair_s[i] = pair;
        src_s[i] = a_div > 0 ? pair / a_div : row;
    }
    __syncthreads();
    const uint16_t* we = w + (size_t)e * N * K;
    mfloatx16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    // PF register sets of loads are on their way while a tile is multiplied: a tile's trip from memory takes longer
    // than the multiplication of one tile, and a block has nothing else to do meanwhile.
    constexpr int PF = 3;
    uint4 ra[PF][A_CH], rw[PF][W_CH];
    size_t arow[A_CH];
#pragma unroll
    for (int i = 0; i < A_CH; i++) arow[i] = (size_t)src_s[(tid + i * NT) / CPR] * lda;
    auto gload = [&](uint4* ra, uint4* rw, int k0) {
#pragma unroll
        for (int i = 0; i < A_CH; i++) {
            const int c = tid + i * NT, kk = k0 + (c % CPR) * 8;
            ra[i] = kk < K ? *reinterpret_cast<const uint4*>(a + arow[i] + kk) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < W_CH; i++) {
            const int c = tid + i * NT, row = c / CPR, kk = k0 + (c % CPR) * 8;
            int n = n0 + row;
            n = n < N ? n : N - 1;
            rw[i] = kk < K ? *reinterpret_cast<const uint4*>(we + (size_t)n * K + kk) : make_uint4(0, 0, 0, 0);
        }
    };
    auto sstore = [&](int stage, const uint4* ra, const uint4* rw) {
        uint16_t* sa = smem + stage * STAGE;
        uint16_t* sw = sa + BM * STRIDE;
#pragma unroll
        for (int i = 0; i < A_CH; i++) {
            const int c = tid + i * NT;
            *reinterpret_cast<uint4*>(sa + (c / CPR) * STRIDE + (c % CPR) * 8) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_CH; i++) {
            const int c = tid + i * NT;
            *reinterpret_cast<uint4*>(sw + (c / CPR) * STRIDE + (c % CPR) * 8) = rw[i];
        }
    };
    auto compute = [&](int stage) {
        const uint16_t* sa = smem + stage * STAGE + (wm * TM + (lane & 31)) * STRIDE + (lane >> 5) * 8;
        const uint16_t* sw = smem + stage * STAGE + (BM + wn * TN + (lane & 31)) * STRIDE + (lane >> 5) * 8;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            MFrag fa[FM], fw[FN];
#pragma unroll
            for (int j = 0; j < FN; j++) fw[j].u = *reinterpret_cast<const uint4*>(sw + j * 32 * STRIDE + kk);
#pragma unroll
            for (int i = 0; i < FM; i++) {
                // an expert's last tile is seldom full: a wave multiplies only the runs of 32 rows that hold any
                if (wm * TM + 32 * i >= nr) continue;
                fa[i].u = *reinterpret_cast<const uint4*>(sa + i * 32 * STRIDE + kk);
#pragma unroll
                for (int j = 0; j < FN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i].v, fw[j].v, acc[i][j], 0, 0, 0);
            }
        }
    };
    const int nk = (K + BK - 1) / BK;
#pragma unroll
    for (int p = 0; p < PF; p++)
        if (p < nk) gload(ra[p], rw[p], p * BK);
    sstore(0, ra[0], rw[0]);
    if (PF < nk) gload(ra[0], rw[0], PF * BK);
    __syncthreads();
    for (int t0 = 0; t0 < nk; t0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {                       // tile t0 + p: the register sets are constants here
            const int t = t0 + p;
            if (t >= nk) break;
            compute(t & 1);
            if (t + 1 < nk) {
                sstore((t + 1) & 1, ra[(p + 1) % PF], rw[(p + 1) % PF]);
                if (t + 1 + PF < nk) gload(ra[(p + 1) % PF], rw[(p + 1) % PF], (t + 1 + PF) * BK);
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int i = 0; i < FM; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = wm * TM + 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
            if (row >= nr) continue;
            const int pair = pair_s[row];
            const float sc = pair_scale ? pair_scale[pair] : 1.f;
            const size_t orow = out_by_pair ? (size_t)pair : (size_t)(r0 + row);
            if (gated) {                                    // (FN is even: blocks 2 j and 2 j + 1 of a wave's columns are gate and up)
#pragma unroll
                for (int j = 0; j + 1 < FN; j += 2) {
                    const int nb = n0 + wn * TN + 32 * j;              // a multiple of 64: TN is
                    if (nb + 32 + (lane & 31) < N)
                        out[orow * ldo + nb / 2 + (lane & 31)] = from_f32<TO>(gated_apply(acc[i][j][r], acc[i][j + 1][r], sc, ga));
                }
                continue;
            }
#pragma unroll
            for (int j = 0; j < FN; j++) {
                const int n = n0 + wn * TN + 32 * j + (lane & 31);
                if (n < N) out[orow * ldo + n] = from_f32<TO>(hfa_act_apply(act, acc[i][j][r]) * sc);
            }
        }
    }
}

extern "C" int hfa_moe_tile_rows(int dtype, int w_dtype, int n_pairs, int n_experts, int N, int K) {
    if (dtype == HFA_BF16 && w_dtype == HFA_BF16 && K % 16 == 0 && N % 32 == 0)
        return n_pairs >= 96 * n_experts ? 128 : n_pairs >= 48 * n_experts ? 64 : 32;
    return PM;
}

extern "C" int hfa_moe_gemm(const void* a, int lda, int dtype, int a_div, const void* w, int w_dtype, const int* row_pair,
                            const int* tiles, const int* n_tiles, int max_tiles, int tile_rows, void* out, int ldo,
                            int out_dtype, int out_by_pair, const float* pair_scale, int act, int N, int K,
                            int force_plain, int gated, float gate_alpha, float gate_limit, float gate_shift, hipStream_t stream) {
    HFA_REQUIRE(a && w && row_pair && tiles && n_tiles && out && max_tiles > 0 && N > 0 && K > 0 && lda >= K &&
                    ldo >= (gated ? N / 2 : N), "moe_gemm: bad arguments");
    HFA_REQUIRE(!gated || (N % 64 == 0 && act == 0), "moe_gemm: gated experts come in blocks of 32 gate rows and 32 up rows, without another activation");
    const GatedAct ga = {gate_alpha, gate_limit, gate_shift};
    HFA_REQUIRE((dtype == HFA_F32 || dtype == HFA_BF16) && (out_dtype == HFA_F32 || out_dtype == HFA_BF16) &&
                    (w_dtype == HFA_F32 || w_dtype == HFA_BF16), "moe_gemm: unknown dtype");
    HFA_REQUIRE(act >= 0 && act <= HFA_ACT_LAST && a_div >= 0, "moe_gemm: bad activation or divisor");
    const bool mfma = !force_plain && dtype == HFA_BF16 && w_dtype == HFA_BF16 && K % 16 == 0 && N % 32 == 0 && lda % 8 == 0 &&
                      (tile_rows == 32 || tile_rows == 64 || tile_rows == 128) && ((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0;
    if (mfma && tile_rows >= 64) {
        // (tiles of 128 x 256, on four waves and on eight, were measured and are slower at every size tried)
        const int n_col_tiles = (N + 127) / 128;
        HFA_REQUIRE((long)max_tiles * n_col_tiles + 8 < (1L << 31), "moe_gemm: too many tiles");
        dim3 grid(((max_tiles * n_col_tiles + 7) / 8 + 1) * 8);      // every XCD's run of units has room, whatever the tile count
#define MOE_LDS(BM, BN, BK, WM, WN, TO)                                                                                   \
    do {                                                                                                                  \
        auto kernel = moe_gemm_lds_kernel<BM, BN, BK, WM, WN, TO>;                                                        \
        constexpr int SMEM = 2 * (BM + BN) * (BK + 8) * 2;                                                                \
        static bool configured = false;                                                                                   \
        if (!configured) {                                                                                                \
            if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM) != hipSuccess) {  \
                hfa_set_error("moe_gemm: cannot reserve %d bytes of LDS", SMEM);                                          \
                return 2;                                                                                                 \
            }                                                                                                             \
            configured = true;                                                                                            \
        }                                                                                                                 \
        kernel<<<grid, WM * WN * WAVE, SMEM, stream>>>((const uint16_t*)a, lda, a_div, (const uint16_t*)w, row_pair, tiles, n_tiles,     \
                                                       (TO*)out, ldo, out_by_pair, pair_scale, act, N, K, n_col_tiles, gated, ga);   \
    } while (0)
        if (tile_rows == 128) { if (out_dtype == HFA_F32) MOE_LDS(128, 128, 32, 2, 2, float); else MOE_LDS(128, 128, 32, 2, 2, bf16); }
        else { if (out_dtype == HFA_F32) MOE_LDS(64, 128, 32, 2, 2, float); else MOE_LDS(64, 128, 32, 2, 2, bf16); }
#undef MOE_LDS
    } else if (mfma && K % 64 == 0) {
        dim3 grid(max_tiles, gated ? N / 64 : (N + 31) / 32);
#define MOE_SPLIT(TO, GATED)                                                                                              \
    moe_gemm_split_kernel<TO, GATED><<<grid, 256, 0, stream>>>((const uint16_t*)a, lda, a_div, (const uint16_t*)w, row_pair, tiles, \
                                                               n_tiles, (TO*)out, ldo, out_by_pair, pair_scale, act, N, K, ga)
        if (out_dtype == HFA_F32) { if (gated) MOE_SPLIT(float, true); else MOE_SPLIT(float, false); }
        else { if (gated) MOE_SPLIT(bf16, true); else MOE_SPLIT(bf16, false); }
#undef MOE_SPLIT
    } else if (mfma) {
        const int cn = gated || (N % 256 == 0 && N >= 512) ? 2 : 1;
        dim3 grid(max_tiles, (N + 128 * cn - 1) / (128 * cn));
#define MOE_ARGS (const uint16_t*)a, lda, a_div, (const uint16_t*)w, row_pair, tiles, n_tiles
#define MOE_TAIL ldo, out_by_pair, pair_scale, act, N, K, gated, ga
#define MOE_GO(RM, CN)                                                                                                  \
    do {                                                                                                                \
        if (out_dtype == HFA_F32) moe_gemm_mfma_kernel<RM, CN, float><<<grid, 256, 0, stream>>>(MOE_ARGS, (float*)out, MOE_TAIL); \
        else moe_gemm_mfma_kernel<RM, CN, bf16><<<grid, 256, 0, stream>>>(MOE_ARGS, (bf16*)out, MOE_TAIL);                  \
    } while (0)
        if (cn == 2) MOE_GO(1, 2); else MOE_GO(1, 1);
#undef MOE_GO
#undef MOE_ARGS
#undef MOE_TAIL
    } else {
        HFA_REQUIRE(tile_rows <= PM, "moe_gemm: the plain kernel takes tiles of at most %d rows, got %d", PM, tile_rows);
        dim3 grid(max_tiles, (N + PN - 1) / PN);
#define MOE_PLAIN(TA, TW, TO)                                                                                          \
    moe_gemm_plain_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>((const TA*)a, lda, a_div, (const TW*)w, row_pair, tiles, n_tiles, \
                                                                  (TO*)out, ldo, out_by_pair, pair_scale, act, N, K, gated, ga)
        if (dtype == HFA_F32 && w_dtype == HFA_F32 && out_dtype == HFA_F32) MOE_PLAIN(float, float, float);
        else if (dtype == HFA_BF16 && w_dtype == HFA_BF16 && out_dtype == HFA_F32) MOE_PLAIN(bf16, bf16, float);
        else if (dtype == HFA_BF16 && w_dtype == HFA_BF16 && out_dtype == HFA_BF16) MOE_PLAIN(bf16, bf16, bf16);
        else if (dtype == HFA_BF16 && w_dtype == HFA_F32 && out_dtype == HFA_F32) MOE_PLAIN(bf16, float, float);
        else if (dtype == HFA_BF16 && w_dtype == HFA_F32 && out_dtype == HFA_BF16) MOE_PLAIN(bf16, float, bf16);
        else
            HFA_REQUIRE(false, "moe_gemm: this mix of operand and result types is not taken (fp32 activations go with fp32 matrices and results)");
#undef MOE_PLAIN
    }
    HFA_LAUNCH_CHECK("moe_gemm");
    return 0;
}

// ---- the weighted sum -----------------------------------------------------------------------
// x[t, :] += y[t * top, :] + ... + y[t * top + top - 1, :] (fp32; the weights are in y already), choices in order.
__global__ void moe_combine_kernel(const float* __restrict__ y, float* __restrict__ x, int top, int width, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / width, c = i % width;
        float s = 0.f;
        for (int k = 0; k < top; k++) s += y[(t * top + k) * width + c];
        x[i] += s;
    }
}
// the same, four columns a thread (width a multiple of 4)
__global__ void moe_combine4_kernel(const float4* __restrict__ y, float4* __restrict__ x, int top, int width4, size_t total4) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / width4, c = i % width4;
        float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int k = 0; k < top; k++) {
            const float4 v = y[(t * top + k) * width4 + c];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        float4 o = x[i];
        o.x += s.x; o.y += s.y; o.z += s.z; o.w += s.w;
        x[i] = o;
    }
}

extern "C" int hfa_moe_combine(const float* y, float* x, int n_tokens, int top, int width, hipStream_t stream) {
    HFA_REQUIRE(y && x && n_tokens > 0 && top > 0 && width > 0, "moe_combine: bad arguments");
    const bool vec = width % 4 == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)x & 15) == 0;
    const size_t total = (size_t)n_tokens * width / (vec ? 4 : 1);
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (vec) moe_combine4_kernel<<<blocks, 256, 0, stream>>>((const float4*)y, (float4*)x, top, width / 4, total);
    else moe_combine_kernel<<<blocks, 256, 0, stream>>>(y, x, top, width, total);
    HFA_LAUNCH_CHECK("moe_combine");
    return 0;
}

// ---- gated experts ------------------------------------------------------------------------
// Row r of the expert-ordered rows holds [gate: F | up: F] fp32 sums of one (token, choice) pair. With c = pair_scale of
// the row's pair (null: 1), g = min(c gate, limit), u = clamp(c up, -limit, limit) (limit <= 0: no bounds):
// mid[r, f] = g sigmoid(alpha g) (u + shift). Scaling the sums is scaling the expert's input. `interleaved`: the row holds
// blocks of 32 gate sums and 32 up sums instead (F a multiple of 32).
template <typename TO>
__global__ void moe_gated_act_kernel(const float* __restrict__ gu, int ld, const int* __restrict__ row_pair,
                                     const float* __restrict__ pair_scale, TO* __restrict__ out, int ldo, int F, float alpha,
                                     float limit, float shift, int interleaved, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / F, f = i % F;
        const float c = pair_scale ? pair_scale[row_pair[r]] : 1.f;
        const size_t gi = interleaved ? (f / 32) * 64 + f % 32 : f, ui = interleaved ? gi + 32 : F + f;
        float g = c * gu[r * ld + gi], u = c * gu[r * ld + ui];
        if (limit > 0.f) {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
        }
        out[r * ldo + f] = from_f32<TO>(g / (1.0f + expf(-alpha * g)) * (u + shift));
    }
}

extern "C" int hfa_moe_gated_act(const float* gu, int ld, const int* row_pair, const float* pair_scale, void* out,
                                 int out_dtype, int ldo, int n_rows, int F, float alpha, float limit, float shift,
                                 int interleaved, hipStream_t stream) {
    HFA_REQUIRE(gu && out && n_rows > 0 && F > 0 && ld >= 2 * F && ldo >= F && (!pair_scale || row_pair) && (!interleaved || F % 32 == 0),
                "moe_gated_act: bad arguments");
    HFA_REQUIRE(out_dtype == HFA_F32 || out_dtype == HFA_BF16, "moe_gated_act: unknown dtype %d", out_dtype);
    const size_t total = (size_t)n_rows * F;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (out_dtype == HFA_F32)
        moe_gated_act_kernel<float><<<blocks, 256, 0, stream>>>(gu, ld, row_pair, pair_scale, (float*)out, ldo, F, alpha, limit, shift, interleaved, total);
    else
        moe_gated_act_kernel<bf16><<<blocks, 256, 0, stream>>>(gu, ld, row_pair, pair_scale, (bf16*)out, ldo, F, alpha, limit, shift, interleaved, total);
    HFA_LAUNCH_CHECK("moe_gated_act");
    return 0;
}
