// Layer norm with scale and shift, the RMS norm in groups (with a gate), the activations of the plain feed-forward layers (erf gelu, tanh gelu,
// squared relu) and the soft cap of the logits.
#include "api.h"
#include "common.h"

#define LN_PLANE_BATCH 8

// ---- layer norm -------------------------------------------------------------------------
// out[r, :] = (x - mean) / sqrt(var + eps) * w + b, var = the mean squared deviation, all in fp32. One block a
// row; mean and variance are summed in a fixed order in two passes over the row (the deviations are formed from
// the finished mean, so a row far from zero loses nothing), and a row's result does not depend on the rest of the
// launch. As in hfa_rmsnorm, a product that left its result as partial sums (the residual sum of the layer before)
// is finished first: x[r, :] += sum over splits + bias, written back.
#define LN_KEEP 8          // values of the row that a thread keeps in registers between the passes
template <typename TO>
__global__ __launch_bounds__(1024) void layernorm_kernel(float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, TO* __restrict__ out,
                                                        const int* __restrict__ rows, int width, float eps,
                                                        const float* __restrict__ partial, int splits,
                                                        const float* __restrict__ pbias, int n_rows) {
    __shared__ float red[17];
    const int r = blockIdx.x, bd = blockDim.x;
    const int xr = rows ? rows[r] : r;
    float* src = x + (size_t)xr * width;
    // the row's value at column i, with a deferred product's partial sums added (and written back) first
    auto value = [&](int i) {
        float v = src[i];
        if (splits > 0) {
            for (int s0 = 0; s0 < splits; s0 += LN_PLANE_BATCH) {
                float p[LN_PLANE_BATCH];
#pragma unroll
                for (int u = 0; u < LN_PLANE_BATCH; u++)
                    p[u] = s0 + u < splits ? partial[((size_t)(s0 + u) * n_rows + xr) * width + i] : 0.f;
#pragma unroll
                for (int u = 0; u < LN_PLANE_BATCH; u++) v += p[u];
            }
            if (pbias) v += pbias[i];
            src[i] = v;
        }
        return v;
    };
    // Rows of up to LN_KEEP values a thread are read once; what lies beyond is read again in each pass.
    float keep[LN_KEEP];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < LN_KEEP; k++) {
        const int i = threadIdx.x + k * bd;
        keep[k] = i < width ? value(i) : 0.f;
        sum += keep[k];
    }
    for (int i = threadIdx.x + LN_KEEP * bd; i < width; i += bd) sum += value(i);
    const float mean = block_sum(sum, red) / (float)width;      // the barriers inside also order the writes of x
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < LN_KEEP; k++) {
        const float d = keep[k] - mean;
        if ((int)threadIdx.x + k * bd < width) sq = fmaf(d, d, sq);
    }
    for (int i = threadIdx.x + LN_KEEP * bd; i < width; i += bd) {
        const float d = src[i] - mean;
        sq = fmaf(d, d, sq);
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)width + eps);
    TO* dst = out + (size_t)r * width;
#pragma unroll
    for (int k = 0; k < LN_KEEP; k++) {
        const int i = threadIdx.x + k * bd;
        if (i < width) dst[i] = from_f32<TO>(fmaf((keep[k] - mean) * inv, w[i], b ? b[i] : 0.f));
    }
    for (int i = threadIdx.x + LN_KEEP * bd; i < width; i += bd)
        dst[i] = from_f32<TO>(fmaf((src[i] - mean) * inv, w[i], b ? b[i] : 0.f));
}

extern "C" int hfa_layernorm(float* x, const float* w, const float* b, void* out, int out_dtype, const int* rows,
                             int n_rows, int width, float eps, const float* partial, int splits,
                             const float* partial_bias, int x_rows, hipStream_t stream) {
    HFA_REQUIRE(x && w && out && n_rows > 0 && width > 0, "layernorm: bad arguments");
    HFA_REQUIRE(out_dtype == HFA_F32 || out_dtype == HFA_BF16, "layernorm: unknown dtype %d", out_dtype);
    HFA_REQUIRE(splits == 0 || (partial && !rows), "layernorm: partial sums go with all rows in order");
    const int threads = width >= 8192 ? 1024 : width >= 2048 ? 512 : width >= 512 ? 256 : width >= 128 ? 128 : 64;
    if (out_dtype == HFA_F32)
        layernorm_kernel<float><<<n_rows, threads, 0, stream>>>(x, w, b, (float*)out, rows, width, eps, partial, splits,
                                                                partial_bias, x_rows);
    else
        layernorm_kernel<bf16><<<n_rows, threads, 0, stream>>>(x, w, b, (bf16*)out, rows, width, eps, partial, splits,
                                                               partial_bias, x_rows);
    HFA_LAUNCH_CHECK("layernorm");
    return 0;
}

// ---- activations ------------------------------------------------------------------------
template <typename T>
__global__ void activation_kernel(const T* __restrict__ in, int ldi, T* __restrict__ out, int ldo, int width, int kind,
                                  size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / width, c = i % width;
        out[r * ldo + c] = from_f32<T>(hfa_act_apply(kind, to_f32(in[r * ldi + c])));
    }
}

extern "C" int hfa_activation(const void* in, int ldi, void* out, int ldo, int dtype, int n_rows, int width, int kind,
                              hipStream_t stream) {
    HFA_REQUIRE(in && out && n_rows > 0 && width > 0 && ldi >= width && ldo >= width, "activation: bad arguments");
    HFA_REQUIRE(kind >= HFA_ACT_GELU_ERF && kind <= HFA_ACT_LAST, "activation: unknown kind %d", kind);
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "activation: unknown dtype %d", dtype);
    const size_t total = (size_t)n_rows * width;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (dtype == HFA_F32)
        activation_kernel<float><<<blocks, 256, 0, stream>>>((const float*)in, ldi, (float*)out, ldo, width, kind, total);
    else
        activation_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)in, ldi, (bf16*)out, ldo, width, kind, total);
    HFA_LAUNCH_CHECK("activation");
    return 0;
}

// ---- soft cap ---------------------------------------------------------------------------
// x <- cap * tanh(x / cap), fp32, in place.
__global__ void softcap_kernel(float* __restrict__ x, int ld, int width, float cap, float inv_cap, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        float* p = x + (i / width) * ld + i % width;
        *p = cap * tanhf(*p * inv_cap);
    }
}

extern "C" int hfa_softcap(float* x, int ld, int n_rows, int width, float cap, hipStream_t stream) {
    HFA_REQUIRE(x && n_rows > 0 && width > 0 && ld >= width && cap > 0.f, "softcap: bad arguments");
    const size_t total = (size_t)n_rows * width;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    softcap_kernel<<<blocks, 256, 0, stream>>>(x, ld, width, cap, 1.0f / cap, total);
    HFA_LAUNCH_CHECK("softcap");
    return 0;
}

// ---- RMS norm in groups, with an optional gate ----------------------------------------------
// A row of `width` values is cut into `groups` equal runs; each run is divided by sqrt(mean(run^2) + eps) and the
// whole is multiplied by w (one block a (row, run); sums in fp32 in a fixed order). gate_kind 1: the row is first
// multiplied by silu(gate) (the gate comes before the norm); gate_kind 2: the normed and weighted row is multiplied
// by sigmoid(gate) (the gate comes after); gate_kind 3: by silu(gate), also after. `rows`: out[r] is the norm of x[rows[r]] (the gate's rows are not gathered).
template <typename TX, typename TG, typename TO>
__global__ __launch_bounds__(1024) void group_rmsnorm_kernel(const TX* __restrict__ x, int ldx, const float* __restrict__ w,
                                                            TO* __restrict__ out, int ldo, const int* __restrict__ rows,
                                                            int run, float eps, const TG* __restrict__ gate, int ldg,
                                                            int gate_kind, const float* __restrict__ row_scale) {
    __shared__ float red[17];
    const int r = blockIdx.x, c0 = blockIdx.y * run;
    const float pre = row_scale ? row_scale[(size_t)r * gridDim.y + blockIdx.y] : 1.f;     // a factor of this (row, run), before the norm
    const TX* src = x + (size_t)(rows ? rows[r] : r) * ldx + c0;
    const TG* gsrc = gate ? gate + (size_t)r * ldg + c0 : nullptr;
    constexpr int KEEP = 4;
    float keep[KEEP];
    auto value = [&](int i) {
        float v = to_f32(src[i]) * pre;
        if (gate_kind == 1) {
            const float z = to_f32(gsrc[i]);
            v *= z / (1.0f + expf(-z));
        }
        return v;
    };
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        const int i = threadIdx.x + k * blockDim.x;
        keep[k] = i < run ? value(i) : 0.f;
        ss = fmaf(keep[k], keep[k], ss);
    }
    for (int i = threadIdx.x + KEEP * blockDim.x; i < run; i += blockDim.x) {
        const float v = value(i);
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)run + eps);
    TO* dst = out + (size_t)r * ldo + c0;
    auto finish = [&](int i, float v) {
        float y = v * inv * w[c0 + i];
        if (gate_kind == 2) y *= 1.0f / (1.0f + expf(-to_f32(gsrc[i])));
        if (gate_kind == 3) { const float z = to_f32(gsrc[i]); y *= z / (1.0f + expf(-z)); }
        dst[i] = from_f32<TO>(y);
    };
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        const int i = threadIdx.x + k * blockDim.x;
        if (i < run) finish(i, keep[k]);
    }
    for (int i = threadIdx.x + KEEP * blockDim.x; i < run; i += blockDim.x) finish(i, value(i));
}

extern "C" int hfa_group_rmsnorm(const void* x, int x_dtype, int ldx, const float* w, void* out, int out_dtype, int ldo,
                                 const int* rows, int n_rows, int width, int groups, float eps, const void* gate,
                                 int gate_dtype, int ldg, int gate_kind, const float* row_scale, hipStream_t stream) {
    HFA_REQUIRE(!row_scale || !rows, "group_rmsnorm: factors per (row, run) go with rows in order");
    HFA_REQUIRE(x && w && out && n_rows > 0 && width > 0 && ldx >= width && ldo >= width, "group_rmsnorm: bad arguments");
    HFA_REQUIRE(groups > 0 && width % groups == 0 && groups <= 65535, "group_rmsnorm: %d values do not form %d equal runs", width, groups);
    HFA_REQUIRE((x_dtype == HFA_F32 || x_dtype == HFA_BF16) && (out_dtype == HFA_F32 || out_dtype == HFA_BF16),
                "group_rmsnorm: unknown dtype");
    HFA_REQUIRE(gate_kind >= 0 && gate_kind <= 3 && (gate_kind == 0 || (gate && ldg >= width && !rows &&
                                                                       (gate_dtype == HFA_F32 || gate_dtype == HFA_BF16))),
                "group_rmsnorm: a gate needs its rows, one for each row in order");
    const int run = width / groups;
    const int threads = run >= 4096 ? 1024 : run >= 1024 ? 256 : run >= 256 ? 128 : 64;
    dim3 grid(n_rows, groups);
#define GRN(TX, TG, TO)                                                                                                 \
    group_rmsnorm_kernel<TX, TG, TO><<<grid, threads, 0, stream>>>((const TX*)x, ldx, w, (TO*)out, ldo, rows, run, eps, \
                                                                   (const TG*)(gate_kind ? gate : nullptr), ldg, gate_kind, row_scale)
    const bool gb = gate_kind && gate_dtype == HFA_BF16;
    if (x_dtype == HFA_F32 && out_dtype == HFA_F32) { if (gb) GRN(float, bf16, float); else GRN(float, float, float); }
    else if (x_dtype == HFA_F32) { if (gb) GRN(float, bf16, bf16); else GRN(float, float, bf16); }
    else if (out_dtype == HFA_F32) { if (gb) GRN(bf16, bf16, float); else GRN(bf16, float, float); }
    else { if (gb) GRN(bf16, bf16, bf16); else GRN(bf16, float, bf16); }
#undef GRN
    HFA_LAUNCH_CHECK("group_rmsnorm");
    return 0;
}

// ---- a branch's result on its way into the stream, and a gate on a mixer's heads ---------------------
// hfa_scale_add: out[r, c] (+)= scale * col[c] * y[r, c] in fp32 (col null: 1): a residual sum whose branch is multiplied by
// one number and, column by column, by a learned vector.
__global__ void scale_add_kernel(const float* __restrict__ y, int ldy, const float* __restrict__ col, float scale,
                                 float* __restrict__ out, int ldo, int width, int accumulate, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / width, c = i % width;
        const float v = (col ? scale * col[c] : scale) * y[r * ldy + c];
        float* o = out + r * ldo + c;
        *o = accumulate ? *o + v : v;
    }
}

extern "C" int hfa_scale_add(const float* y, int ldy, const float* col, float scale, float* out, int ldo, int n_rows, int width,
                             int accumulate, hipStream_t stream) {
    HFA_REQUIRE(y && out && n_rows > 0 && width > 0 && ldy >= width && ldo >= width, "scale_add: bad arguments");
    const size_t total = (size_t)n_rows * width;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    scale_add_kernel<<<blocks, 256, 0, stream>>>(y, ldy, col, scale, out, ldo, width, accumulate, total);
    HFA_LAUNCH_CHECK("scale_add");
    return 0;
}

// hfa_gate_mul: out[r, c] = x[r, c] * act(gate[r, c]), the product formed in fp32 (act: HFA_ACT_SIGMOID or HFA_ACT_SILU).
template <typename TX, typename TG, typename TO>
__global__ void gate_mul_kernel(const TX* __restrict__ x, int ldx, const TG* __restrict__ gate, int ldg, TO* __restrict__ out,
                                int ldo, int width, int act, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / width, c = i % width;
        out[r * ldo + c] = from_f32<TO>(to_f32(x[r * ldx + c]) * hfa_act_apply(act, to_f32(gate[r * ldg + c])));
    }
}

extern "C" int hfa_gate_mul(const void* x, int x_dtype, int ldx, const void* gate, int gate_dtype, int ldg, void* out, int out_dtype,
                            int ldo, int n_rows, int width, int act, hipStream_t stream) {
    HFA_REQUIRE(x && gate && out && n_rows > 0 && width > 0 && ldx >= width && ldg >= width && ldo >= width, "gate_mul: bad arguments");
    HFA_REQUIRE(act == HFA_ACT_SIGMOID || act == HFA_ACT_SILU, "gate_mul: the gate's function is the logistic function or silu");
    HFA_REQUIRE((x_dtype == HFA_F32 || x_dtype == HFA_BF16) && (gate_dtype == HFA_F32 || gate_dtype == HFA_BF16) &&
                    (out_dtype == HFA_F32 || out_dtype == HFA_BF16), "gate_mul: unknown dtype");
    const size_t total = (size_t)n_rows * width;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
#define GM(TX, TG, TO) gate_mul_kernel<TX, TG, TO><<<blocks, 256, 0, stream>>>((const TX*)x, ldx, (const TG*)gate, ldg, (TO*)out, ldo, width, act, total)
    const bool xb = x_dtype == HFA_BF16, gb = gate_dtype == HFA_BF16, ob = out_dtype == HFA_BF16;
    if (xb && gb && ob) GM(bf16, bf16, bf16);
    else if (!xb && !gb && !ob) GM(float, float, float);
    else if (!xb && gb && ob) GM(float, bf16, bf16);
    else if (!xb && !gb && ob) GM(float, float, bf16);
    else if (xb && !gb && ob) GM(bf16, float, bf16);
    else { hfa_set_error("gate_mul: this mix of dtypes is not built"); return 1; }
#undef GM
    HFA_LAUNCH_CHECK("gate_mul");
    return 0;
}
