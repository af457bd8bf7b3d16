// Decoded tokens of a mixer that mixes its heads' attention weights after the softmax: every head's weights applied to
// the values of EVERY key/value group, in one pass over the cache (bf16 cache, fp32 scores, softmax and sums).
//
// hfa_talk_mix wants A(h, c) = softmax_h . V_c for all heads h and groups c. Pass by pass (one attention call a round of
// groups) the cache is read G times; here a token's keys and values are read once:
//
//   a block owns one token and one chunk of its keys (and, from six groups on, one half of the groups' values); its NDB waves all hold the same 32 "columns", the token's heads
//   (H <= 32), and each wave owns 32 of a value head's D = 32 NDB dimensions in every group.
//   S^T[key, col] = sum over groups g and dims d of K[key, g, d] . Q'[col, g, d], where Q' is the head's query in the
//   slot of its own group and zero in the others: one chain of G D / 16 products v_mfma_f32_32x32x16_bf16 (A = 32 keys x
//   16 dims straight from the cache, B = queries in registers, zeroed where the group is not the column's) gives every
//   head its score against the keys of its own group. The waves of a block share the chain out by groups and add their
//   sums through LDS, so every wave holds all scores.
//   online softmax per column (a lane pair), as in attention_mfma.hip; the probabilities a lane holds are the B operand of
//   O_c^T[dim, col] += V_c^T[dim, key] . P^T[key, col]      for every group c, dims of the wave's slice
//
// Each wave leaves (max, sum) and its unnormalised slice for its chunk; attn_cross_merge_kernel puts the chunks together
// and writes [T][G rounds][H][D], round r of head h being its weights on the values of group (c(h) + r) mod G.
#include "attention_internal.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define KB 32
#define CROSS_PG_MAX 1024
#define CROSS_MAX_CHUNKS 64
#define NEG_BIG (-1.0e30f)
#define MAX_SLACK 8.0f

namespace {

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float pair_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t prob_pair(float lo, float hi) {
    const floatx2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

union Frag {
    uint4 u;
    uint2 h[2];
    bf16x8 v;
};

// partial: [token][chunk] records of [H][G][D] unnormalised outputs followed by H (max, sum) pairs, padded to whole float4s
__host__ __device__ __forceinline__ size_t cross_record(int H, int G, int D) { return (size_t)H * G * D + (size_t)((2 * H + 3) / 4 * 4); }

template <int NDB, int NG, int NV>
__global__ __launch_bounds__(NDB * WAVE) void attn_cross_decode_kernel(
    const uint16_t* __restrict__ q, int ldq, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc, int kvw,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_slot, const int* __restrict__ positions,
    float* __restrict__ partial, int H, int psh, float scale_log2e, int chunk_keys, int n_chunks) {
    constexpr int D = NDB * 32, KS = D / 16;
    const int P = 1 << psh;
    const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5, slice = threadIdx.x >> 6;
    const int tok = blockIdx.x, chunk = blockIdx.y, v0 = blockIdx.z * NV;      // the block's value groups: v0 .. v0 + NV - 1
    const int hi = positions[tok];                          // the token's own position: its last key
    const int k_begin = chunk * chunk_keys;                 // a multiple of the key block
    if (k_begin > hi) return;                               // the merge counts the chunks that hold keys from the position
    const int k_end = hi < k_begin + chunk_keys - 1 ? hi : k_begin + chunk_keys - 1;
    const bool col_ok = col < H;
    const int cpt = H / NG;                                 // heads of a group
    const int my_grp = col_ok ? col / cpt : -1;
    const int* bt = block_table + (size_t)token_slot[tok] * max_blocks;

    __shared__ int pg_s[CROSS_PG_MAX];
    const int pw0 = k_begin >> psh;
    {
        const int n_pg = (k_end >> psh) - pw0 + 1;           // at most CROSS_PG_MAX (the launcher's choice of chunk_keys)
        for (int i = threadIdx.x; i < n_pg; i += NDB * WAVE) pg_s[i] = bt[pw0 + i];
    }
    Frag qf[KS];
    {
        const uint16_t* qp = q + (size_t)tok * ldq + (col_ok ? col : 0) * D + half * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            qf[ks].u = col_ok ? *reinterpret_cast<const uint4*>(qp + ks * 16) : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    auto page_of = [&](int key) { return pg_s[(key >> psh) - pw0]; };

    auto load_k = [&](int key0, int g, Frag (&kf)[KS]) {
        int key = key0 + col;
        key = key < k_end ? key : k_end;                   // rows past the end repeat the last key; they are masked
        const int page = page_of(key);
        const unsigned off = __umul24((unsigned)((page << psh) + (key & (P - 1))), (unsigned)kvw) + (unsigned)(g * D + half * 8);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kf[ks].u = *reinterpret_cast<const uint4*>(kc + (off + (unsigned)(ks * 16)));
    };
    // values of a block, for product step kk: keys key0 + 16 kk + 4 half + {0..3} and the same + 8, dimension
    // 32 slice + col of every group
    auto load_v = [&](int key0, Frag (&vf)[NV][2]) {
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int run = 0; run < 2; run++) {
                int ka = key0 + 16 * kk + 8 * run + 4 * half;
                ka = ka < (k_end & ~3) ? ka : (k_end & ~3);
                const int page = page_of(ka);
                const unsigned off = __umul24((unsigned)(page << psh), (unsigned)kvw) + (unsigned)(((32 * slice + col) << psh) + (ka & (P - 1)));
#pragma unroll
                for (int c = 0; c < NV; c++)
                    vf[c][kk].h[run] = *reinterpret_cast<const uint2*>(vc + (off + (unsigned)(((v0 + c) * D) << psh)));
            }
        }
    };

    floatx16 o[NV];
#pragma unroll
    for (int c = 0; c < NV; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[c][r] = 0.f;
    float m = NEG_BIG, l = 0.f;
    const uint4 zero4 = make_uint4(0, 0, 0, 0);

    // The chain over the groups is shared out: wave w forms the products of the groups w, w + NDB, ... (columns of other
    // groups get zeros there), the waves leave their sums in LDS and every wave adds all of them, in the order of the
    // waves, so all hold the same scores. Two sets of sums in turn, so one barrier a key block is enough.
    constexpr int NJ = (NG + NDB - 1) / NDB;               // groups a wave, at most
    __shared__ float st_s[2][NDB][16][WAVE];
    const int nb = (k_end - k_begin) / KB + 1;
    Frag kf[NJ][KS], vf[NV][2];
    auto load_k_mine = [&](int key0) {
#pragma unroll
        for (int j = 0; j < NJ; j++)
            if (slice + j * NDB < NG) load_k(key0, slice + j * NDB, kf[j]);
    };
    load_k_mine(k_begin);
    for (int b = 0; b < nb; b++) {
        const int key0 = k_begin + b * KB;
        load_v(key0, vf);
        floatx16 st;
#pragma unroll
        for (int r = 0; r < 16; r++) st[r] = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            if (slice + j * NDB < NG) {                     // (the same for the whole wave)
                const bool mine = my_grp == slice + j * NDB;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    Frag b_op;
                    b_op.u = mine ? qf[ks].u : zero4;
                    st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[j][ks].v, b_op.v, st, 0, 0, 0);
                }
            }
        }
        if (b + 1 < nb) load_k_mine(key0 + KB);             // the next block's keys are on their way from here on
        if (NDB > 1) {
#pragma unroll
            for (int r = 0; r < 16; r++) st_s[b & 1][slice][r][lane] = st[r];
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float sum = st_s[b & 1][0][r][lane];
#pragma unroll
                for (int w = 1; w < NDB; w++) sum += st_s[b & 1][w][r][lane];
                st[r] = sum;
            }
        }
        // element r of the lane: key key0 + 8 (r / 4) + 4 half + r % 4, this lane's column
        float mx = NEG_BIG, mn, corr, psum = 0.f;
        const bool inside = key0 + KB - 1 <= k_end;
        if (inside) {
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[r]);
            mx = pair_max(mx) * scale_log2e;
            mn = mx > m + MAX_SLACK ? mx : m;
            corr = fast_exp2(m - mn);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                st[r] = fast_exp2(fmaf(st[r], scale_log2e, -mn));
                psum += st[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int kr = key0 + 8 * (r / 4) + 4 * half + (r % 4);
                st[r] = kr <= k_end ? st[r] * scale_log2e : NEG_BIG;
                mx = fmaxf(mx, st[r]);
            }
            mx = pair_max(mx);
            mn = mx > m + MAX_SLACK ? mx : m;
            corr = fast_exp2(m - mn);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float p = st[r] > 0.5f * NEG_BIG ? fast_exp2(st[r] - mn) : 0.f;
                st[r] = p;
                psum += p;
            }
            // what the cache holds past the last key is not this request's (Inf and NaN included, and 0 x Inf is NaN)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int run = 0; run < 2; run++) {
                    const int k4 = key0 + 16 * kk + 8 * run + 4 * half;
                    uint32_t mk[2];
#pragma unroll
                    for (int e = 0; e < 2; e++)
                        mk[e] = (k4 + 2 * e <= k_end ? 0x0000ffffu : 0u) | (k4 + 2 * e + 1 <= k_end ? 0xffff0000u : 0u);
#pragma unroll
                    for (int c = 0; c < NV; c++) {
                        vf[c][kk].h[run].x &= mk[0];
                        vf[c][kk].h[run].y &= mk[1];
                    }
                }
        }
        psum = pair_sum(psum);
        l = l * corr + psum;
        m = mn;
        if (__any(corr != 1.0f)) {
#pragma unroll
            for (int c = 0; c < NV; c++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[c][r] *= corr;
        }
        Frag pf[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = prob_pair(st[8 * kk + 2 * e], st[8 * kk + 2 * e + 1]);
            pf[kk].u = make_uint4(w[0], w[1], w[2], w[3]);
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int c = 0; c < NV; c++)
                o[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[c][kk].v, pf[kk].v, o[c], 0, 0, 0);
    }

    if (!col_ok) return;
    // element r of o[c]: dimension 32 slice + 8 (r / 4) + 4 half + r % 4 of group v0 + c, this lane's column
    float* rec = partial + ((size_t)tok * n_chunks + chunk) * cross_record(H, NG, D);
    if (slice == 0 && half == 0 && v0 == 0) {
        rec[H * NG * D + 2 * col] = m;
        rec[H * NG * D + 2 * col + 1] = l;
    }
    float* dst = rec + (size_t)col * NG * D + v0 * D + 32 * slice + 4 * half;
#pragma unroll
    for (int c = 0; c < NV; c++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++)
            *reinterpret_cast<float4*>(dst + c * D + 8 * rg) = make_float4(o[c][4 * rg], o[c][4 * rg + 1], o[c][4 * rg + 2], o[c][4 * rg + 3]);
}

// One block a (token, head): the chunks' records merged in chunk order, normalised, and written in rounds of groups. A thread
// owns four neighbouring dimensions of one group.
__global__ __launch_bounds__(128) void attn_cross_merge_kernel(const float* __restrict__ partial, const int* __restrict__ positions,
                                                              uint16_t* __restrict__ out, int ldo, int H, int G, int D,
                                                              int chunk_keys, int n_chunks) {
    __shared__ float w_s[CROSS_MAX_CHUNKS];
    __shared__ float inv_s;
    const int tok = blockIdx.x, h = blockIdx.y;
    const int live = positions[tok] / chunk_keys + 1;      // the chunks that hold keys of this token (at most CROSS_MAX_CHUNKS = a wave)
    const size_t rec = cross_record(H, G, D);
    const float* src = partial + (size_t)tok * n_chunks * rec;
    if (threadIdx.x < WAVE) {
        const int c = threadIdx.x;
        const float* ml = src + (size_t)H * G * D + 2 * h;
        const float mc = c < live ? ml[c * rec] : NEG_BIG;
        const float M = wave_max(mc);
        const float w = c < live ? exp2f(mc - M) : 0.f;
        const float L = wave_sum(c < live ? w * ml[c * rec + 1] : 0.f);
        if (c < live) w_s[c] = w;
        if (c == 0) inv_s = 1.0f / L;
    }
    __syncthreads();
    const int per = H / G, GD = G * D;
    const float* mine = src + (size_t)h * GD;
    for (int i = 4 * threadIdx.x; i < GD; i += 4 * blockDim.x) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
        for (int k = 0; k < live; k++) {
            const float4 v = *reinterpret_cast<const float4*>(mine + k * rec + i);
            const float w = w_s[k];
            acc.x = fmaf(w, v.x, acc.x);
            acc.y = fmaf(w, v.y, acc.y);
            acc.z = fmaf(w, v.z, acc.z);
            acc.w = fmaf(w, v.w, acc.w);
        }
        const int c = i / D, d = i % D;
        const int r = (c - h / per + G) % G;
        const float inv = inv_s;
        uint2 o;
        o.x = (uint32_t)bf16_bits(acc.x * inv) | ((uint32_t)bf16_bits(acc.y * inv) << 16);
        o.y = (uint32_t)bf16_bits(acc.z * inv) | ((uint32_t)bf16_bits(acc.w * inv) << 16);
        *reinterpret_cast<uint2*>(out + (size_t)tok * ldo + ((size_t)r * H + h) * D + d) = o;
    }
}

int cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
    }
    return n;
}

template <int NDB, int NG, int NV>
int launch(const AttnArgs& a, int chunk_keys, int n_chunks, int psh) {
    attn_cross_decode_kernel<NDB, NG, NV><<<dim3(a.n_tokens, n_chunks, NG / NV), NDB * WAVE, 0, a.stream>>>(
        (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, a.kv_width, a.block_table, a.max_blocks,
        a.token_slot, a.positions, (float*)a.workspace, a.n_heads, psh, a.scale * 1.4426950408889634f, chunk_keys, n_chunks);
    HFA_LAUNCH_CHECK("attn_cross_decode");
    return 0;
}

template <int NDB>
int launch_groups(const AttnArgs& a, int chunk_keys, int n_chunks, int psh) {
    switch (a.n_kv_heads) {
        case 1: return launch<NDB, 1, 1>(a, chunk_keys, n_chunks, psh);
        case 2: return launch<NDB, 2, 2>(a, chunk_keys, n_chunks, psh);
        case 3: return launch<NDB, 3, 3>(a, chunk_keys, n_chunks, psh);
        case 4: return launch<NDB, 4, 4>(a, chunk_keys, n_chunks, psh);
        case 6: return launch<NDB, 6, 3>(a, chunk_keys, n_chunks, psh);       // more groups: two blocks share a chunk's values,
        default: return launch<NDB, 8, 4>(a, chunk_keys, n_chunks, psh);      // each forming all scores (the accumulators' registers)
    }
}

}  // namespace

// Whether a step of single tokens goes this way: what the matrix-core kernels take (attn_mfma_supports), at most 32 heads
// in 1, 2, 3, 4, 6 or 8 groups, and a workspace that holds the chunks' records. Leaves the cut of the keys in chunk_keys, n_chunks.
bool attn_cross_supports(const AttnArgs& a, int* chunk_keys, int* n_chunks) {
    if (a.max_q_len != 1 || a.n_tokens != a.n_seqs || a.n_heads > 32 || a.n_kv_heads > 8 || a.n_kv_heads == 5 || a.n_kv_heads == 7 || a.window || a.mask_chunk || a.sink ||
        a.raw || !a.workspace || a.page_tokens < 4 || a.ldo % 4 || ((uintptr_t)a.out & 7) || !attn_mfma_supports(a))
        return false;
    // Enough blocks for two a compute unit, no chunk of fewer than 64 keys, none whose pages outgrow the kernel's table, and
    // no more chunks than the workspace holds records of.
    const int span = a.max_seq_len;
    const int z = a.n_kv_heads > 4 ? 2 : 1;                 // blocks a (token, chunk)
    long want = (2L * cu_count() + (long)a.n_tokens * z - 1) / ((long)a.n_tokens * z);
    const long most = (span + 63) / 64;
    if (want > most) want = most;
    const size_t per_chunk = (size_t)a.n_tokens * cross_record(a.n_heads, a.n_kv_heads, a.head_dim) * sizeof(float);
    if ((size_t)want * per_chunk > a.workspace_bytes) want = (long)(a.workspace_bytes / per_chunk);
    if (want < 1) return false;
    int ck = (int)(((span + want - 1) / want + KB - 1) / KB * KB);
    const int ck_max = ((CROSS_PG_MAX - 2) * a.page_tokens) / KB * KB;
    if (ck > ck_max) ck = ck_max;
    const int n = (span + ck - 1) / ck;
    if (n > CROSS_MAX_CHUNKS || (size_t)n * per_chunk > a.workspace_bytes) return false;
    *chunk_keys = ck;
    *n_chunks = n;
    return true;
}

int attn_cross_launch(const AttnArgs& a, int chunk_keys, int n_chunks) {
    int psh = 0;
    while ((1 << psh) < a.page_tokens) psh++;
    int rc;
    switch (a.head_dim / 32) {
        case 1: rc = launch_groups<1>(a, chunk_keys, n_chunks, psh); break;
        case 2: rc = launch_groups<2>(a, chunk_keys, n_chunks, psh); break;
        case 3: rc = launch_groups<3>(a, chunk_keys, n_chunks, psh); break;
        default: rc = launch_groups<4>(a, chunk_keys, n_chunks, psh); break;
    }
    if (rc) return rc;
    attn_cross_merge_kernel<<<dim3(a.n_tokens, a.n_heads), 128, 0, a.stream>>>((const float*)a.workspace, a.positions, (uint16_t*)a.out, a.ldo, a.n_heads,
                                                              a.n_kv_heads, a.head_dim, chunk_keys, n_chunks);
    HFA_LAUNCH_CHECK("attn_cross_merge");
    return 0;
}
