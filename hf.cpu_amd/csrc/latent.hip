// Attention whose keys and values are expanded from one latent a token: the glue between the projections and the
// attention kernels. With the expansion folded into the queries (q' = Wuk^T q) and taken out of the values (o = Wuv sum p c),
// the cache holds one key/value head a token: key [rotated part | latent], value [latent].
#include "api.h"
#include "common.h"

// One block a token. down[t] = [latent before its norm: C | rotated key part: R] (fp32); q[t] head by head [D | R].
// packed[t] = [H x (R | C) | R | C | C]: the heads' R parts copied (their C parts are written by the products that fold
// the keys' expansion into the queries, or copied from `folded`, [T][H x C] of q's type, if given), the key's R part copied, and
// the normed latent twice.
template <typename TQ, typename TO>
__global__ __launch_bounds__(256) void latent_pack_kernel(const float* __restrict__ down, int ld_down, const TQ* __restrict__ q,
                                                         int ldq, const float* __restrict__ w, float eps, TO* __restrict__ packed,
                                                         int ld_packed, int H, int D, int R, int C, const TQ* __restrict__ folded,
                                                         int ld_folded) {
    __shared__ float red[17];
    const int t = blockIdx.x;
    const float* dr = down + (size_t)t * ld_down;
    float ss = 0.f;
    for (int i = threadIdx.x; i < C; i += blockDim.x) ss = fmaf(dr[i], dr[i], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)C + eps);
    TO* pr = packed + (size_t)t * ld_packed;
    TO* key = pr + (size_t)H * (R + C);
    for (int i = threadIdx.x; i < C; i += blockDim.x) {
        const TO c = from_f32<TO>(dr[i] * inv * w[i]);
        key[R + i] = c;
        key[R + C + i] = c;
    }
    for (int i = threadIdx.x; i < R; i += blockDim.x) key[i] = from_f32<TO>(dr[C + i]);
    const TQ* qr = q + (size_t)t * ldq;
    for (int i = threadIdx.x; i < H * R; i += blockDim.x) {
        const int h = i / R, r = i % R;
        pr[(size_t)h * (R + C) + r] = from_f32<TO>(to_f32(qr[(size_t)h * (D + R) + D + r]));
    }
    if (folded) {
        const TQ* fr = folded + (size_t)t * ld_folded;
        for (int i = threadIdx.x; i < H * C; i += blockDim.x) {
            const int h = i / C, c = i % C;
            pr[(size_t)h * (R + C) + R + c] = from_f32<TO>(to_f32(fr[i]));
        }
    }
}

extern "C" int hfa_latent_pack(const float* down, int ld_down, const void* q, int q_dtype, int ldq, const float* w, float eps,
                               void* packed, int out_dtype, int ld_packed, int n_tokens, int n_heads, int dim, int rot, int latent,
                               const void* folded, int ld_folded, hipStream_t stream) {
    HFA_REQUIRE(down && q && w && packed && n_tokens > 0 && n_heads > 0 && dim > 0 && rot >= 0 && latent > 0, "latent_pack: bad arguments");
    HFA_REQUIRE(ld_down >= latent + rot && ldq >= n_heads * (dim + rot) && ld_packed >= n_heads * (rot + latent) + rot + 2 * latent,
                "latent_pack: a row is shorter than its parts");
    HFA_REQUIRE(!folded || ld_folded >= n_heads * latent, "latent_pack: the folded queries' rows are shorter than the heads' latents");
    HFA_REQUIRE((q_dtype == HFA_F32 || q_dtype == HFA_BF16) && (out_dtype == HFA_F32 || out_dtype == HFA_BF16), "latent_pack: unknown dtype");
#define LP(TQ, TO) latent_pack_kernel<TQ, TO><<<n_tokens, 256, 0, stream>>>(down, ld_down, (const TQ*)q, ldq, w, eps, (TO*)packed, ld_packed, n_heads, dim, rot, latent, (const TQ*)folded, ld_folded)
    if (q_dtype == HFA_F32 && out_dtype == HFA_F32) LP(float, float);
    else if (q_dtype == HFA_BF16 && out_dtype == HFA_BF16) LP(bf16, bf16);
    else if (q_dtype == HFA_F32) LP(float, bf16);
    else LP(bf16, float);
#undef LP
    HFA_LAUNCH_CHECK("latent_pack");
    return 0;
}
