// Parts of layers that norm a sublayer's result before it joins the residual stream, and what such designs bring with
// them: an embedding with a scale and a sinusoidal position vector, the norm of a (gated) branch added into the stream,
// an activation made of normed powers, a scale on fp32 rows, the per-head norm of queries and keys with the store of
// keys and values, and the mixing of attention outputs across heads.
//
//   hfa_embed_pos         x[t] = table[token] * scale + sinusoid(position)
//   hfa_rmsnorm_add       out[r] (+)= scale * rmsnorm(y[r] * sigmoid(gate[r])) * w
//   hfa_polynorm          out = a N(z) + b N(z^2) + c N(z^3) + e, N dividing a row by its root mean square
//   hfa_scale_rows        x *= s
//   hfa_head_norm_store   per head: q, k <- rms or unit norm (a weight of one head's size, shared); q to a matrix, k and
//                         v to their cache rows
//   hfa_talk_mix          out[t, h] = sigmoid(gate[t, h]) * sum_g talk[h, g] * A[t, g, values of h's group]
#include "api.h"
#include "common.h"

// ---- embedding with a scale and a sinusoidal position vector ------------------------------------------------------
// Entry 2i of the position vector is sin(p f_i), entry 2i + 1 cos(p f_i), f_i = base^(-2i / width) (inv_freq, rounded
// from 64-bit on the host); the angle is one fp32 product.
template <typename T>
__global__ void embed_pos_kernel(const T* __restrict__ table, const int* __restrict__ tokens, const int* __restrict__ positions,
                                 const float* __restrict__ inv_freq, float* __restrict__ x, int width, int vocab, float scale) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const T* row = table + (size_t)tok * width;
    float* dst = x + (size_t)t * width;
    const float pos = positions ? (float)positions[t] : 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = to_f32(row[i]) * scale;
        if (positions) {
            const float ang = pos * inv_freq[i >> 1];
            v += (i & 1) ? cosf(ang) : sinf(ang);
        }
        dst[i] = v;
    }
}

extern "C" int hfa_embed_pos(const void* table, int table_dtype, const int* tokens, const int* positions, const float* inv_freq,
                             float* x, int n_tokens, int width, int vocab, float scale, hipStream_t stream) {
    HFA_REQUIRE(table && tokens && x && n_tokens > 0 && width > 0 && vocab > 0, "embed_pos: bad arguments");
    HFA_REQUIRE(!positions || inv_freq, "embed_pos: positions come with their frequencies");
    HFA_REQUIRE(table_dtype == HFA_F32 || table_dtype == HFA_BF16, "embed_pos: unknown dtype %d", table_dtype);
    if (table_dtype == HFA_F32)
        embed_pos_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, tokens, positions, inv_freq, x, width, vocab, scale);
    else
        embed_pos_kernel<bf16><<<n_tokens, 256, 0, stream>>>((const bf16*)table, tokens, positions, inv_freq, x, width, vocab, scale);
    HFA_LAUNCH_CHECK("embed_pos");
    return 0;
}

// ---- the norm of a branch's result, added into the stream -----------------------------------------------------------
// One block a row, all in fp32: v = y * sigmoid(gate) (gate null: v = y); out (+)= scale * v / sqrt(mean(v^2) + eps) * w.
template <typename TG>
__global__ __launch_bounds__(256) void rmsnorm_add_kernel(const float* __restrict__ y, int ldy, const TG* __restrict__ gate, int ldg,
                                                         const float* __restrict__ gate_bias, const float* __restrict__ w,
                                                         float* __restrict__ out, int ldo, int width, float eps, float scale,
                                                         int accumulate) {
    __shared__ float red[17];
    const int r = blockIdx.x;
    const float* src = y + (size_t)r * ldy;
    const TG* gs = gate ? gate + (size_t)r * ldg : nullptr;
    constexpr int KEEP = 8;
    float keep[KEEP];
    auto value = [&](int i) {
        float v = src[i];
        if (gs) {
            const float z = to_f32(gs[i]) + (gate_bias ? gate_bias[i] : 0.f);
            v *= 1.0f / (1.0f + expf(-z));
        }
        return v;
    };
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        const int i = threadIdx.x + k * blockDim.x;
        keep[k] = i < width ? value(i) : 0.f;
        ss = fmaf(keep[k], keep[k], ss);
    }
    for (int i = threadIdx.x + KEEP * blockDim.x; i < width; i += blockDim.x) {
        const float v = value(i);
        ss = fmaf(v, v, ss);
    }
    const float inv = scale / sqrtf(block_sum(ss, red) / (float)width + eps);
    float* dst = out + (size_t)r * ldo;
    auto finish = [&](int i, float v) {
        const float z = v * inv * w[i];
        dst[i] = accumulate ? dst[i] + z : z;
    };
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        const int i = threadIdx.x + k * blockDim.x;
        if (i < width) finish(i, keep[k]);
    }
    for (int i = threadIdx.x + KEEP * blockDim.x; i < width; i += blockDim.x) finish(i, value(i));
}

extern "C" int hfa_rmsnorm_add(const float* y, int ldy, const void* gate, int gate_dtype, int ldg, const float* gate_bias,
                               const float* w, float* out, int ldo, int n_rows, int width, float eps, float scale, int accumulate,
                               hipStream_t stream) {
    HFA_REQUIRE(y && w && out && n_rows > 0 && width > 0 && ldy >= width && ldo >= width && (!gate || ldg >= width),
                "rmsnorm_add: bad arguments");
    HFA_REQUIRE(!gate || gate_dtype == HFA_F32 || gate_dtype == HFA_BF16, "rmsnorm_add: unknown gate dtype %d", gate_dtype);
    HFA_REQUIRE(gate || !gate_bias, "rmsnorm_add: a gate's bias without the gate");
    if (gate && gate_dtype == HFA_BF16)
        rmsnorm_add_kernel<bf16><<<n_rows, 256, 0, stream>>>(y, ldy, (const bf16*)gate, ldg, gate_bias, w, out, ldo, width, eps, scale, accumulate);
    else
        rmsnorm_add_kernel<float><<<n_rows, 256, 0, stream>>>(y, ldy, (const float*)gate, ldg, gate_bias, w, out, ldo, width, eps, scale, accumulate);
    HFA_LAUNCH_CHECK("rmsnorm_add");
    return 0;
}

// ---- an activation of normed powers ----------------------------------------------------------------------------------
// out = a N(z) + b N(z^2) + c N(z^3) + e over a row, N(u) = u / sqrt(mean(u^2) + eps); coef = (a, b, c, e) on the device.
// The three sums of squares (of z, z^2 and z^3) are taken in one pass, in fp32, in a fixed order.
template <typename TI, typename TO>
__global__ __launch_bounds__(1024) void polynorm_kernel(const TI* __restrict__ z, int ldz, const float* __restrict__ coef,
                                                      TO* __restrict__ out, int ldo, int width, float eps) {
    __shared__ float red[17];
    const int r = blockIdx.x;
    const TI* src = z + (size_t)r * ldz;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll 4
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = to_f32(src[i]), v2 = v * v, v3 = v2 * v;
        s1 = fmaf(v, v, s1);
        s2 = fmaf(v2, v2, s2);
        s3 = fmaf(v3, v3, s3);
    }
    const float n = (float)width;
    const float i1 = coef[0] / sqrtf(block_sum(s1, red) / n + eps);
    const float i2 = coef[1] / sqrtf(block_sum(s2, red) / n + eps);
    const float i3 = coef[2] / sqrtf(block_sum(s3, red) / n + eps);
    const float e = coef[3];
    TO* dst = out + (size_t)r * ldo;
#pragma unroll 4
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = to_f32(src[i]), v2 = v * v;
        dst[i] = from_f32<TO>(v * i1 + v2 * i2 + v2 * v * i3 + e);
    }
}

extern "C" int hfa_polynorm(const void* z, int z_dtype, int ldz, const float* coef, void* out, int out_dtype, int ldo, int n_rows,
                            int width, float eps, hipStream_t stream) {
    HFA_REQUIRE(z && coef && out && n_rows > 0 && width > 0 && ldz >= width && ldo >= width, "polynorm: bad arguments");
    HFA_REQUIRE((z_dtype == HFA_F32 || z_dtype == HFA_BF16) && (out_dtype == HFA_F32 || out_dtype == HFA_BF16), "polynorm: unknown dtype");
    const int threads = width >= 4096 ? 1024 : 256;       // few rows in a decode step: a wide row is shared by more threads
#define PN(TI, TO) polynorm_kernel<TI, TO><<<n_rows, threads, 0, stream>>>((const TI*)z, ldz, coef, (TO*)out, ldo, width, eps)
    if (z_dtype == HFA_F32) { if (out_dtype == HFA_F32) PN(float, float); else PN(float, bf16); }
    else { if (out_dtype == HFA_F32) PN(bf16, float); else PN(bf16, bf16); }
#undef PN
    HFA_LAUNCH_CHECK("polynorm");
    return 0;
}

// ---- x *= s on fp32 rows ---------------------------------------------------------------------------------------------
__global__ void scale_rows_kernel(float* __restrict__ x, int ld, int width, float s, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        float* p = x + (i / width) * ld + i % width;
        *p = *p * s;
    }
}

extern "C" int hfa_scale_rows(float* x, int ld, int n_rows, int width, float s, hipStream_t stream) {
    HFA_REQUIRE(x && n_rows > 0 && width > 0 && ld >= width, "scale_rows: bad arguments");
    const size_t total = (size_t)n_rows * width;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    scale_rows_kernel<<<blocks, 256, 0, stream>>>(x, ld, width, s, total);
    HFA_LAUNCH_CHECK("scale_rows");
    return 0;
}

// ---- queries and keys normed head by head; keys and values to the cache ------------------------------------------------
// Rows [q: H D | k: G D | v: G Dv] (fp32 or bf16): every q head and every k head is divided by sqrt(mean(head^2) + eps) and
// multiplied by a weight of D values that all heads share (q_w, k_w; null: no norm for that part). q goes to q_out
// ([T, H D], the cache's dtype), k to cache row slot_map[t], v to the same row with the page transposed
// ([page][column][offset]). One wave a head, four waves a block, a block a token and four heads; the blocks of a token
// share its values out.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void head_norm_store_kernel(const TI* __restrict__ qkv, int ld, int H, int G, int D, int Dv,
                                                             const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
                                                             TO* __restrict__ q_out, int ldq, TO* __restrict__ k_cache,
                                                             TO* __restrict__ v_cache, const int* __restrict__ slot_map, int page_tokens) {
    const int t = blockIdx.x, lane = threadIdx.x & (WAVE - 1), wv = threadIdx.x / WAVE, nw = blockDim.x / WAVE;
    const TI* row = qkv + (size_t)t * ld;
    const int QD = H * D, KD = G * D, VD = G * Dv;
    const int slot = slot_map[t];
    const int hs = blockIdx.y * nw + wv;
    if (hs < H + G) {
        const bool is_key = hs >= H;
        const TI* src = row + hs * D;
        const float* w = is_key ? k_w : q_w;
        float inv = 1.f;
        if (w) {
            float ss = 0.f;
            for (int i = lane; i < D; i += WAVE) { const float v = to_f32(src[i]); ss = fmaf(v, v, ss); }
            inv = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
        }
        TO* dst = is_key ? k_cache + (size_t)slot * KD + (hs - H) * D : q_out + (size_t)t * ldq + hs * D;
        for (int i = lane; i < D; i += WAVE) {
            float v = to_f32(src[i]);
            if (w) v = v * inv * w[i];
            dst[i] = from_f32<TO>(v);
        }
    }
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < VD; c += gridDim.y * blockDim.x)
        v_cache[(size_t)(slot / page_tokens) * page_tokens * VD + (size_t)c * page_tokens + slot % page_tokens] =
            from_f32<TO>(to_f32(row[QD + KD + c]));
}

extern "C" int hfa_head_norm_store(const void* qkv, int in_dtype, int ld, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                                   const float* q_w, const float* k_w, float eps, void* q_out, int ldq, void* k_cache, void* v_cache,
                                   int out_dtype, const int* slot_map, int page_tokens, int n_tokens, hipStream_t stream) {
    HFA_REQUIRE(qkv && q_out && k_cache && v_cache && slot_map && n_tokens > 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0 &&
                    v_head_dim > 0 && page_tokens > 0, "head_norm_store: bad arguments");
    HFA_REQUIRE(ld >= (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_head_dim && ldq >= n_heads * head_dim,
                "head_norm_store: a row is shorter than its heads");
    HFA_REQUIRE((in_dtype == HFA_F32 || in_dtype == HFA_BF16) && (out_dtype == HFA_F32 || out_dtype == HFA_BF16),
                "head_norm_store: unknown dtype");
#define HNS(TI, TO)                                                                                                          \
    head_norm_store_kernel<TI, TO><<<dim3(n_tokens, (n_heads + n_kv_heads + 3) / 4), 256, 0, stream>>>((const TI*)qkv, ld, n_heads, n_kv_heads, head_dim, v_head_dim, \
                                                                 q_w, k_w, eps, (TO*)q_out, ldq, (TO*)k_cache, (TO*)v_cache,   \
                                                                 slot_map, page_tokens)
    if (in_dtype == HFA_F32) { if (out_dtype == HFA_F32) HNS(float, float); else HNS(float, bf16); }
    else { if (out_dtype == HFA_F32) HNS(bf16, float); else HNS(bf16, bf16); }
#undef HNS
    HFA_LAUNCH_CHECK("head_norm_store");
    return 0;
}

// ---- attention weights mixed across heads, as a sum of attention outputs ------------------------------------------------
// Mixing the heads' softmax weights, weight_h <- sum_g talk[h, g] weight_g, before head h applies them to the values of its
// own group c(h) is, by linearity, out_h = sum_g talk[h, g] A(g, c(h)), where A(g, c) is what head g's weights give on the
// values of group c. `cross` holds these: [T][G rounds][H heads][Dv], round r of head g being its weights on the values
// of group (c(g) + r) mod G (hfa_paged_attention with cross_values). gate (null: none): out is multiplied by
// sigmoid(gate[t, h Dv + d]). Sums in fp32 in the order of g.
// A block a (token, head): with few tokens (a decode step) there are still heads x tokens blocks to fill the machine.
template <typename TA, typename TG, typename TO>
__global__ __launch_bounds__(128) void talk_mix_kernel(const TA* __restrict__ cross, const float* __restrict__ talk,
                                                      const TG* __restrict__ gate, int ldg, TO* __restrict__ out, int ldo, int H,
                                                      int G, int Dv) {
    extern __shared__ float talk_s[];                      // row h of the mix, and where each head's round for h's group lies
    int* at_s = reinterpret_cast<int*>(talk_s + H);
    const int t = blockIdx.x, h = blockIdx.y, per = H / G, c = h / per;
    for (int g = threadIdx.x; g < H; g += blockDim.x) {
        talk_s[g] = talk[h * H + g];
        at_s[g] = (((c - g / per + G) % G) * H + g) * Dv;
    }
    __syncthreads();
    const TA* A = cross + (size_t)t * G * H * Dv;
    for (int d = threadIdx.x; d < Dv; d += blockDim.x) {
        float acc = 0.f;
#pragma unroll 4
        for (int g = 0; g < H; g++) acc = fmaf(talk_s[g], to_f32(A[at_s[g] + d]), acc);
        const int i = h * Dv + d;
        if (gate) acc *= 1.0f / (1.0f + expf(-to_f32(gate[(size_t)t * ldg + i])));
        out[(size_t)t * ldo + i] = from_f32<TO>(acc);
    }
}

extern "C" int hfa_talk_mix(const void* cross, int cross_dtype, const float* talk, const void* gate, int gate_dtype, int ldg, void* out,
                            int out_dtype, int ldo, int n_tokens, int n_heads, int n_kv_heads, int v_head_dim, hipStream_t stream) {
    HFA_REQUIRE(cross && talk && out && n_tokens > 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && v_head_dim > 0,
                "talk_mix: bad arguments");
    HFA_REQUIRE(n_heads <= 128, "talk_mix: %d heads (at most 128)", n_heads);
    HFA_REQUIRE(ldo >= n_heads * v_head_dim && (!gate || ldg >= n_heads * v_head_dim), "talk_mix: a row is shorter than its heads");
    const size_t lds = (size_t)n_heads * (sizeof(float) + sizeof(int));
    const int code = (cross_dtype == HFA_BF16 ? 4 : 0) + ((gate && gate_dtype == HFA_BF16) ? 2 : 0) + (out_dtype == HFA_BF16 ? 1 : 0);
#define TM(TA, TG, TO)                                                                                                          \
    talk_mix_kernel<TA, TG, TO><<<dim3(n_tokens, n_heads), 128, lds, stream>>>((const TA*)cross, talk, (const TG*)gate, ldg, (TO*)out, ldo, n_heads, \
                                                                n_kv_heads, v_head_dim)
    switch (code) {
        case 0: TM(float, float, float); break;
        case 1: TM(float, float, bf16); break;
        case 2: TM(float, bf16, float); break;
        case 3: TM(float, bf16, bf16); break;
        case 4: TM(bf16, float, float); break;
        case 5: TM(bf16, float, bf16); break;
        case 6: TM(bf16, bf16, float); break;
        default: TM(bf16, bf16, bf16); break;
    }
#undef TM
    HFA_LAUNCH_CHECK("talk_mix");
    return 0;
}
