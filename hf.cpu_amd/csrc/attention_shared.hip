// Paged softmax attention of many query heads on ONE key/value head whose key rows are wide (up to 576 values: a latent
// and a rotated part side by side) and whose value rows have a size of their own (up to 512: the latent), bf16 on the
// matrix cores, for prompt portions and decoded tokens alike. This is what attention through latents comes to once the
// keys' expansion is folded into the queries (see hfa_latent_pack): every head reads the same rows.
//
// A block of four waves owns a tile of 32 columns, a column being a (token, head) pair of one request (the tokens of a
// tile are consecutive), and walks the keys of its chunk 32 at a time. The scores' chain of products over the key row is
// shared out between the waves: wave w takes the steps of 16 values w, w + 4, ... of the row, with its part of the
// queries in registers for the whole walk, and the four partial sums meet in LDS (two sets in turn, one barrier a key
// block), added in wave order by every wave, so that all hold the same scores, run the same online softmax and form the
// same probabilities. The value row is shared out too: wave w owns the blocks of 32 value dimensions w, w + 4, ... and
// multiplies the probabilities into them. Keys and values are each read once a tile (keys as rows, values from their
// pages' transposed layout, four keys of a dimension at a time). Fragment conventions are attn_mfma_kernel's: element r
// of a lane's scores is key 8 (r / 4) + 4 half + r % 4 of the block in the lane's column; element r of an accumulator is
// value dimension 8 (r / 4) + 4 half + r % 4 of its block.
//
// Few tiles and long contexts (decoded tokens): the keys are cut into chunks over blockIdx.z, every chunk leaves
// (maximum, sum, unscaled output) and attn_shared_merge_kernel puts them together.
#include "api.h"
#include "common.h"
#include "attention_internal.h"

typedef __bf16 sh_bf16x8 __attribute__((ext_vector_type(8)));
typedef float sh_floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 sh_bf16x2 __attribute__((ext_vector_type(2)));
typedef float sh_floatx2 __attribute__((ext_vector_type(2)));

#define SH_KB 32
#define SH_NEG_BIG (-1.0e30f)
#define SH_MAX_CHUNKS 64

union ShFrag {
    uint4 u;
    uint2 h[2];
    sh_bf16x8 v;
};

__device__ __forceinline__ float sh_pair_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sh_pair_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ uint32_t sh_prob_pair(float lo, float hi) {
    const sh_floatx2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, sh_bf16x2));
}

// KSW: steps of 16 key values a wave takes (4 KSW x 16 >= the key row); NDBW: blocks of 32 value dimensions a wave owns.
template <int KSW, int NDBW, bool SPLIT>
__global__ __launch_bounds__(4 * WAVE) void attn_shared_kernel(
    const uint16_t* __restrict__ q, int ldq, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc, int DK, int C,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_slot, const int* __restrict__ positions,
    const int* __restrict__ q_start, int n_seqs, uint16_t* __restrict__ out, int ldo, float* __restrict__ partial, int H, int psh,
    float scale_log2e, int tpt, int cpt, int chunk_keys, int n_chunks, int one_tile_each) {
    __shared__ float part_s[2][4][16][WAVE];
    const int P = 1 << psh;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE, col = lane & 31, half = lane >> 5;
    const int head0 = blockIdx.y * 32, chunk = blockIdx.z;

    int tile = blockIdx.x, t0 = -1, t_end = 0;
    if (one_tile_each) {
        if (tile < n_seqs) {
            t0 = q_start[tile];
            t_end = q_start[tile + 1];
        }
    } else
    for (int s = 0; s < n_seqs; s++) {
        const int a = q_start[s], b = q_start[s + 1];
        const int nt = (b - a + tpt - 1) / tpt;
        if (tile < nt) {
            t0 = a + tile * tpt;
            t_end = t0 + tpt < b ? t0 + tpt : b;
            break;
        }
        tile -= nt;
    }
    if (t0 < 0 || t_end <= t0) return;                     // the grid is an upper bound on the tiles (uniform over the block)

    const int my_head = head0 + col % cpt;
    const bool col_ok = col < (t_end - t0) * cpt && my_head < H;
    const int my_tok = col_ok ? t0 + col / cpt : t0;
    const int pos = positions[my_tok];
    const int hi = positions[t_end - 1];
    int k_begin = 0, k_end = hi;
    if (SPLIT) {
        k_begin = chunk * chunk_keys;
        k_end = k_end < k_begin + chunk_keys - 1 ? k_end : k_begin + chunk_keys - 1;
    }
    const int vlo = k_begin, vhi = col_ok ? (pos < k_end ? pos : k_end) : -1;
    const int* bt = block_table + (size_t)token_slot[t0] * max_blocks;

    ShFrag qf[KSW];
#pragma unroll
    for (int j = 0; j < KSW; j++) {
        const int ks = wave + 4 * j;
        qf[j].u = (col_ok && ks * 16 < DK) ? *reinterpret_cast<const uint4*>(q + (size_t)my_tok * ldq + (size_t)my_head * DK + ks * 16 + half * 8)
                                           : make_uint4(0, 0, 0, 0);
    }
    sh_floatx16 o[NDBW];
#pragma unroll
    for (int j = 0; j < NDBW; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[j][r] = 0.f;
    float m = SH_NEG_BIG, l = 0.f;

    // this lane's row of a key block (rows past the end repeat the last key; they are masked)
    auto load_k = [&](int key0, ShFrag (&kf)[KSW]) {
        int key = key0 + col;
        key = key < hi ? key : hi;
        const size_t row = ((size_t)bt[key >> psh] << psh) + (key & (P - 1));
        const uint16_t* kp = kc + row * DK + half * 8;
#pragma unroll
        for (int j = 0; j < KSW; j++) {
            const int ks = wave + 4 * j;
            kf[j].u = ks * 16 < DK ? *reinterpret_cast<const uint4*>(kp + ks * 16) : make_uint4(0, 0, 0, 0);
        }
    };
    // The keys of the next block are asked for before this block's products begin, and this block's values as soon as its
    // scores' partial sums are on their way to LDS: the trips to memory run beside the exchange, the softmax and the products.
    int it = 0;
    const int key_first = (k_begin / SH_KB) * SH_KB;
    ShFrag kf[KSW], kn[KSW];
    if (key_first <= k_end) load_k(key_first, kf);
    for (int key0 = key_first; key0 <= k_end; key0 += SH_KB, it++) {
        load_k(key0 + SH_KB <= k_end ? key0 + SH_KB : key0, kn);
        sh_floatx16 st;
#pragma unroll
        for (int r = 0; r < 16; r++) st[r] = 0.f;
#pragma unroll
        for (int j = 0; j < KSW; j++) st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[j].v, qf[j].v, st, 0, 0, 0);
        const int buf = it & 1;
#pragma unroll
        for (int r = 0; r < 16; r++) part_s[buf][wave][r][lane] = st[r];
        // values: for product step kk the lane needs keys key0 + 16 kk + 8 run + 4 half + {0..3} of dimension 32 db + col
        ShFrag vf[NDBW][2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int run = 0; run < 2; run++) {
                int ka = key0 + 16 * kk + 8 * run + 4 * half;
                ka = ka < (hi & ~3) ? ka : (hi & ~3);       // runs past the end are masked; read a valid one
                const uint16_t* vp = vc + ((size_t)bt[ka >> psh] << psh) * C + (ka & (P - 1));
#pragma unroll
                for (int j = 0; j < NDBW; j++) {
                    const int db = wave + 4 * j;
                    vf[j][kk].h[run] = db * 32 < C ? *reinterpret_cast<const uint2*>(vp + ((size_t)(db * 32 + col) << psh)) : make_uint2(0, 0);
                }
            }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; r++)
            st[r] = ((part_s[buf][0][r][lane] + part_s[buf][1][r][lane]) + part_s[buf][2][r][lane]) + part_s[buf][3][r][lane];

        float mx = SH_NEG_BIG, psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int kr = key0 + 8 * (r / 4) + 4 * half + (r % 4);
            st[r] = (kr >= vlo && kr <= vhi) ? st[r] * scale_log2e : SH_NEG_BIG;
            mx = fmaxf(mx, st[r]);
        }
        mx = sh_pair_max(mx);
        const float mn = fmaxf(m, mx);
        const float corr = __builtin_amdgcn_exp2f(m - mn);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = st[r] > 0.5f * SH_NEG_BIG ? __builtin_amdgcn_exp2f(st[r] - mn) : 0.f;
            st[r] = p;
            psum += p;
        }
        psum = sh_pair_sum(psum);
        l = l * corr + psum;
        m = mn;
        if (__any(corr != 1.0f)) {
#pragma unroll
            for (int j = 0; j < NDBW; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[j][r] *= corr;
        }
        ShFrag pf[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = sh_prob_pair(st[8 * kk + 2 * e], st[8 * kk + 2 * e + 1]);
            pf[kk].u = make_uint4(w[0], w[1], w[2], w[3]);
        }
        // Keys outside [k_begin, k_end] weigh nothing in every column, but what the cache holds there is not this request's
        // (Inf and NaN included, and 0 x Inf is NaN): their values are replaced by zeros. Only the first and the last block
        // of a walk have such keys.
        if (key0 < k_begin || key0 + SH_KB - 1 > k_end) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int run = 0; run < 2; run++) {
                    const int kb = key0 + 16 * kk + 8 * run + 4 * half;
                    uint32_t mk[2];
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const bool lo_ok = kb + 2 * e >= k_begin && kb + 2 * e <= k_end;
                        const bool hi_ok = kb + 2 * e + 1 >= k_begin && kb + 2 * e + 1 <= k_end;
                        mk[e] = (lo_ok ? 0x0000ffffu : 0u) | (hi_ok ? 0xffff0000u : 0u);
                    }
#pragma unroll
                    for (int j = 0; j < NDBW; j++) {
                        vf[j][kk].h[run].x &= mk[0];
                        vf[j][kk].h[run].y &= mk[1];
                    }
                }
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int j = 0; j < NDBW; j++) o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[j][kk].v, pf[kk].v, o[j], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < KSW; j++) kf[j].u = kn[j].u;
    }
    if (!col_ok) return;
    // element r of o[j]: value dimension 32 (wave + 4 j) + 8 (r / 4) + 4 half + r % 4 of this lane's column
    if (SPLIT) {
        float* dst = partial + ((size_t)(my_tok * H + my_head) * n_chunks + chunk) * (C + 2);
        if (wave == 0 && half == 0) {
            dst[0] = m;
            dst[1] = l;
        }
#pragma unroll
        for (int j = 0; j < NDBW; j++) {
            const int db = wave + 4 * j;
            if (db * 32 >= C) continue;
#pragma unroll
            for (int rg = 0; rg < 4; rg++)
#pragma unroll
                for (int e = 0; e < 4; e++) dst[2 + 32 * db + 8 * rg + 4 * half + e] = o[j][4 * rg + e];
        }
    } else {
        const float inv = 1.0f / l;
        uint16_t* dst = out + (size_t)my_tok * ldo + (size_t)my_head * C;
#pragma unroll
        for (int j = 0; j < NDBW; j++) {
            const int db = wave + 4 * j;
            if (db * 32 >= C) continue;
#pragma unroll
            for (int rg = 0; rg < 4; rg++) {
                uint2 v;
                v.x = (uint32_t)bf16_bits(o[j][4 * rg] * inv) | ((uint32_t)bf16_bits(o[j][4 * rg + 1] * inv) << 16);
                v.y = (uint32_t)bf16_bits(o[j][4 * rg + 2] * inv) | ((uint32_t)bf16_bits(o[j][4 * rg + 3] * inv) << 16);
                *reinterpret_cast<uint2*>(dst + 32 * db + 8 * rg + 4 * half) = v;
            }
        }
    }
}

// out[t, h, :] = sum_c o_c 2^(m_c - M) / sum_c l_c 2^(m_c - M), chunks in ascending order. One block a (token, head). The kernel is
// a chain of trips to memory and little else: the chunks' maxima and sums are fetched by one thread each, at once, and a thread's
// values of all chunks are asked for eight at a time before they are added.
__global__ __launch_bounds__(256) void attn_shared_merge_kernel(const float* __restrict__ partial, uint16_t* __restrict__ out, int ldo, int H,
                                                                int C, int n_chunks) {
    __shared__ float m_s[SH_MAX_CHUNKS], l_s[SH_MAX_CHUNKS], w_s[SH_MAX_CHUNKS];
    const int t = blockIdx.x, h = blockIdx.y;
    const size_t row = C + 2;
    const float* src = partial + (size_t)(t * H + h) * n_chunks * row;
    if ((int)threadIdx.x < n_chunks) {
        const float2 ml = *reinterpret_cast<const float2*>(src + threadIdx.x * row);
        m_s[threadIdx.x] = ml.x;
        l_s[threadIdx.x] = ml.y;
    }
    __syncthreads();
    float M = SH_NEG_BIG;
    for (int c = 0; c < n_chunks; c++) M = fmaxf(M, m_s[c]);
    float L = 0.f;
    for (int c = 0; c < n_chunks; c++) {
        const float w = exp2f(m_s[c] - M);
        if (threadIdx.x == 0) w_s[c] = w;
        L = fmaf(l_s[c], w, L);
    }
    __syncthreads();
    const float inv = 1.0f / L;
    for (int d = threadIdx.x; d < C; d += blockDim.x) {
        float acc = 0.f;
        for (int c0 = 0; c0 < n_chunks; c0 += 8) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = c0 + i < n_chunks ? src[(c0 + i) * row + 2 + d] : 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (c0 + i < n_chunks) acc = fmaf(v[i], w_s[c0 + i], acc);
        }
        out[(size_t)t * ldo + (size_t)h * C + d] = bf16_bits(acc * inv);
    }
}

static int sh_page_shift(int page_tokens) {
    int s = 0;
    while ((1 << s) < page_tokens) s++;
    return (1 << s) == page_tokens ? s : -1;
}

bool attn_shared_supports(const AttnArgs& a, int v_head_dim, int v_width) {
    return a.n_kv_heads == 1 && a.head_dim % 16 == 0 && a.head_dim <= 576 && v_head_dim % 32 == 0 && v_head_dim <= 512 &&
           a.kv_width == a.head_dim && v_width == v_head_dim && a.page_tokens >= 4 && sh_page_shift(a.page_tokens) >= 0 && a.scale > 0.f &&
           a.window == 0 && a.mask_chunk == 0 && !a.sink && a.v_rot == 0 && a.weights == 0 && a.softcap == 0.f && a.q_start != nullptr &&
           a.raw == nullptr && a.ldq % 8 == 0 && a.ldo % 4 == 0 && ((uintptr_t)a.q & 15) == 0 && ((uintptr_t)a.out & 7) == 0 &&
           ((uintptr_t)a.k_cache & 15) == 0 && ((uintptr_t)a.v_cache & 15) == 0 && (size_t)a.n_tokens * a.n_heads < ((size_t)1 << 31) / 600;
}

int attn_shared_launch(const AttnArgs& a, int v_head_dim) {
    const int H = a.n_heads, DK = a.head_dim, C = v_head_dim;
    const int cpt = H < 32 ? H : 32, tpt = 32 / cpt, head_blocks = (H + 31) / 32;
    const int one_each = a.max_q_len <= tpt ? 1 : 0;
    const int tiles = one_each ? a.n_seqs : (a.n_tokens + tpt - 1) / tpt + a.n_seqs;
    HFA_REQUIRE(tiles <= 0x7fffffff / 2 && head_blocks <= 65535, "paged_attention: the step exceeds the grid");
    // few blocks and long contexts: cut the keys into chunks so that the machine is full
    int n_chunks = 1, chunk_keys = a.max_seq_len;
    const long blocks = (long)(one_each ? a.n_seqs : (a.n_tokens + tpt - 1) / tpt) * head_blocks;
    if (blocks < 512 && a.max_seq_len > 256 && a.workspace) {
        long want = (512 + blocks - 1) / blocks;
        const long most = (a.max_seq_len + 127) / 128;        // no chunk of fewer than 128 keys (64 were measured: no gain)
        if (want > most) want = most;
        if (want > SH_MAX_CHUNKS) want = SH_MAX_CHUNKS;
        chunk_keys = (int)(((a.max_seq_len + want - 1) / want + SH_KB - 1) / SH_KB * SH_KB);
        n_chunks = (a.max_seq_len + chunk_keys - 1) / chunk_keys;
        const size_t need = (size_t)a.n_tokens * H * n_chunks * (C + 2) * sizeof(float);
        if (n_chunks < 2 || n_chunks > SH_MAX_CHUNKS || need > a.workspace_bytes) {
            n_chunks = 1;
            chunk_keys = a.max_seq_len;
        }
    }
    dim3 grid(tiles, head_blocks, n_chunks);
    const float sl = a.scale * 1.4426950408889634f;
#define SH_ARGS                                                                                                                     \
    (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, DK, C, a.block_table, a.max_blocks,          \
        a.token_slot, a.positions, a.q_start, a.n_seqs, (uint16_t*)a.out, a.ldo, (float*)a.workspace, H, sh_page_shift(a.page_tokens), \
        sl, tpt, cpt, chunk_keys, n_chunks, one_each
#define SH_GO(KSW, NDBW)                                                                               \
    do {                                                                                               \
        if (n_chunks > 1) attn_shared_kernel<KSW, NDBW, true><<<grid, 4 * WAVE, 0, a.stream>>>(SH_ARGS); \
        else attn_shared_kernel<KSW, NDBW, false><<<grid, 4 * WAVE, 0, a.stream>>>(SH_ARGS);           \
    } while (0)
    if (DK <= 192 && C <= 128) SH_GO(3, 1);
    else if (DK <= 320 && C <= 256) SH_GO(5, 2);
    else SH_GO(9, 4);
#undef SH_GO
#undef SH_ARGS
    HFA_LAUNCH_CHECK("attn_shared");
    if (n_chunks > 1) {
        attn_shared_merge_kernel<<<dim3(a.n_tokens, H), 256, 0, a.stream>>>((const float*)a.workspace, (uint16_t*)a.out, a.ldo, H, C, n_chunks);
        HFA_LAUNCH_CHECK("attn_shared_merge");
    }
    return 0;
}
