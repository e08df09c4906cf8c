// Row-wise kernels around a sublayer whose norm sits on its output, and around mixers that run side by side:
//
//   embed_scaled:     r = E[id] * scale (float32), and a copy of r in the activations' format;
//   branch_norm_add:  r += layer_scale * norm(y), the norm (layer norm with gain and bias, or RMS norm with gain) over the
//                     sublayer's output y, which may come as parts of a split product that are added in order;
//                     again with a copy of the new r in the activations' format, which the next sublayer reads
//                     (the sublayers read r itself: there is no norm before them);
//   gate_rows:        out = scale * x * gate(g), element by element, into columns of a wider row (the heads of
//                     several mixers side by side, for one output product);
//   row_norm_gate:    out = scale * x / sqrt(mean(x^2) + eps) * gain * gate(g), the mean over the whole row (all heads
//                     of a mixer together), likewise into columns of a wider row.
//
// The residual, the statistics of every norm, the layer scale and the gates' sigmoids are float32; a value is
// rounded once, when it is stored in the activations' format.  One workgroup a row; a row's sums are taken in an
// order that depends on the row's width alone.
#include "api.h"
#include "common.h"

#define BR_NORM_RMS 1
#define BR_NORM_LAYER 2
#define BR_GATE_SIGMOID 0
#define BR_GATE_SILU 1

template <typename TW, typename TA>
__global__ void __launch_bounds__(256)
embed_scaled_kernel(float* __restrict__ out, TA* __restrict__ act, const TW* __restrict__ table,
                    const int32_t* __restrict__ ids, float scale, int dim) {
    const int t = blockIdx.x;
    const TW* row = table + (size_t)ids[t] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = to_f32(row[d]) * scale;
        out[(size_t)t * dim + d] = v;
        if (act) from_f32(act + (size_t)t * dim + d, v);
    }
}

extern "C" int ri_embed_scaled(float* out, void* act, int act_dtype, const void* table, int table_dtype, const int32_t* ids,
                               float scale, int tokens, int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && dim > 0, "embed_scaled: tokens %d, dim %d", tokens, dim);
    RI_REQUIRE((table_dtype == RI_F32 || table_dtype == RI_BF16) && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "embed_scaled: table dtype %d, activations %d", table_dtype, act_dtype);
    hipStream_t s = (hipStream_t)stream;
#define RI_GO(TW, TA) embed_scaled_kernel<TW, TA><<<tokens, 256, 0, s>>>(out, (TA*)act, (const TW*)table, ids, scale, dim)
    if (table_dtype == RI_F32) { if (act_dtype == RI_F32) RI_GO(float, float); else RI_GO(float, bf16_t); }
    else                       { if (act_dtype == RI_F32) RI_GO(bf16_t, float); else RI_GO(bf16_t, bf16_t); }
#undef RI_GO
    RI_LAUNCH_CHECK("embed_scaled");
    return 0;
}

// The row's y is kept in LDS as float32 between the passes (parts added once, in order).
template <typename TY, typename TA>
__global__ void __launch_bounds__(256)
branch_norm_add_kernel(float* __restrict__ residual, TA* __restrict__ act, const TY* __restrict__ y, int parts,
                       size_t part_stride, const float* __restrict__ gain, const float* __restrict__ bias, float eps,
                       int kind, const float* __restrict__ layer_scale, int dim) {
    extern __shared__ float row[];                           // dim floats
    __shared__ float scratch[16];
    const size_t at = (size_t)blockIdx.x * dim;
    float sum = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = to_f32(y[at + d]);
        for (int p = 1; p < parts; ++p) v += to_f32(y[p * part_stride + at + d]);
        row[d] = v;
        sum += v;
    }
    float mean = 0.f;
    if (kind == BR_NORM_LAYER) mean = block_sum(sum, scratch) / (float)dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float c = row[d] - mean;
        ss += c * c;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = (row[d] - mean) * inv * gain[d];
        if (bias) v += bias[d];
        if (layer_scale) v *= layer_scale[d];
        const float r = residual[at + d] + v;
        residual[at + d] = r;
        if (act) from_f32(act + at + d, r);
    }
}

extern "C" int ri_branch_norm_add(float* residual, void* act, int act_dtype, const void* y, int y_dtype, int parts,
                                  const float* gain, const float* bias, float eps, int kind, const float* layer_scale,
                                  int rows, int dim, void* stream) {
    RI_REQUIRE(rows > 0 && dim > 0 && parts >= 1, "branch_norm_add: %d rows of %d in %d parts", rows, dim, parts);
    RI_REQUIRE(kind == BR_NORM_RMS || kind == BR_NORM_LAYER, "branch_norm_add: norm kind %d", kind);
    RI_REQUIRE(gain && residual && y, "branch_norm_add: a gain, a residual and a branch output are needed");
    RI_REQUIRE((size_t)dim * sizeof(float) <= 64 * 1024, "branch_norm_add: rows of %d exceed the kernel's 16384", dim);
    RI_REQUIRE((y_dtype == RI_F32 || y_dtype == RI_BF16) && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "branch_norm_add: dtypes %d and %d", y_dtype, act_dtype);
    RI_REQUIRE(parts == 1 || y_dtype == RI_F32, "branch_norm_add: parts of a product are float32");
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)dim * sizeof(float), stride = (size_t)rows * dim;
#define RI_GO(TY, TA)                                                                                                   \
    branch_norm_add_kernel<TY, TA><<<rows, 256, lds, s>>>(residual, (TA*)act, (const TY*)y, parts, stride, gain, bias, eps, \
                                                         kind, layer_scale, dim)
    if (lds > 48 * 1024) {
        static bool asked = false;
        if (!asked) {
            hipFuncSetAttribute((const void*)branch_norm_add_kernel<float, float>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
            hipFuncSetAttribute((const void*)branch_norm_add_kernel<float, bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
            hipFuncSetAttribute((const void*)branch_norm_add_kernel<bf16_t, float>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
            hipFuncSetAttribute((const void*)branch_norm_add_kernel<bf16_t, bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
            asked = true;
        }
    }
    if (y_dtype == RI_F32) { if (act_dtype == RI_F32) RI_GO(float, float); else RI_GO(float, bf16_t); }
    else                   { if (act_dtype == RI_F32) RI_GO(bf16_t, float); else RI_GO(bf16_t, bf16_t); }
#undef RI_GO
    RI_LAUNCH_CHECK("branch_norm_add");
    return 0;
}

__device__ __forceinline__ float gate_of(float g, int kind) {
    const float sg = 1.0f / (1.0f + expf(-g));
    return kind == BR_GATE_SILU ? g * sg : sg;
}

template <typename TX, typename TA>
__global__ void __launch_bounds__(256)
gate_rows_kernel(TA* __restrict__ out, int out_stride, const TX* __restrict__ x, const TA* __restrict__ gate, int gate_stride,
                 float scale, int kind, int width) {
    const size_t t = blockIdx.x;
    for (int d = threadIdx.x; d < width; d += blockDim.x)
        from_f32(out + t * out_stride + d,
                 scale * to_f32(x[t * width + d]) * (gate ? gate_of(to_f32(gate[t * gate_stride + d]), kind) : 1.0f));
}

// out[t, out_off + d] = scale * x[t, d] * gate(g[t, g_off + d]); x: [rows, width] in its own format; g and out share
// the activations' format.  gate NULL: the scaled copy alone.
extern "C" int ri_gate_rows(void* out, int out_stride, int out_off, const void* x, int x_dtype, const void* gate,
                            int gate_stride, int g_off, int act_dtype, float scale, int kind, int rows, int width,
                            void* stream) {
    RI_REQUIRE(rows > 0 && width > 0, "gate_rows: %d rows of %d", rows, width);
    RI_REQUIRE(out_off >= 0 && out_off + width <= out_stride && (!gate || (g_off >= 0 && g_off + width <= gate_stride)),
               "gate_rows: columns %d..+%d of rows of %d, gates %d..+%d of rows of %d", out_off, width, out_stride, g_off,
               width, gate_stride);
    RI_REQUIRE(kind == BR_GATE_SIGMOID || kind == BR_GATE_SILU, "gate_rows: gate kind %d", kind);
    RI_REQUIRE((x_dtype == RI_F32 || x_dtype == RI_BF16) && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "gate_rows: dtypes %d and %d", x_dtype, act_dtype);
    hipStream_t s = (hipStream_t)stream;
#define RI_GO(TX, TA)                                                                                                  \
    gate_rows_kernel<TX, TA><<<rows, 256, 0, s>>>((TA*)out + out_off, out_stride, (const TX*)x,                             \
                                                  gate ? (const TA*)gate + g_off : nullptr,                              \
                                                  gate_stride, scale, kind, width)
    if (x_dtype == RI_F32) { if (act_dtype == RI_F32) RI_GO(float, float); else RI_GO(float, bf16_t); }
    else                   { if (act_dtype == RI_F32) RI_GO(bf16_t, float); else RI_GO(bf16_t, bf16_t); }
#undef RI_GO
    RI_LAUNCH_CHECK("gate_rows");
    return 0;
}

template <typename TA>
__global__ void __launch_bounds__(256)
row_norm_gate_kernel(TA* __restrict__ out, int out_stride, const float* __restrict__ x, const float* __restrict__ gain,
                     float eps, const TA* __restrict__ gate, int gate_stride, float scale, int kind, int width) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    float ss = 0.f;
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        const float v = x[t * width + d];
        ss += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        float v = x[t * width + d] * inv;
        if (gain) v *= gain[d];
        if (gate) v *= gate_of(to_f32(gate[t * gate_stride + d]), kind);
        from_f32(out + t * out_stride + d, scale * v);
    }
}

// out[t, out_off + d] = scale * x[t, d] / sqrt(mean_d(x[t, :]^2) + eps) * gain[d] * gate(g[t, g_off + d]); x float32.
extern "C" int ri_row_norm_gate(void* out, int out_stride, int out_off, const float* x, const float* gain, float eps,
                                const void* gate, int gate_stride, int g_off, int act_dtype, float scale, int kind,
                                int rows, int width, void* stream) {
    RI_REQUIRE(rows > 0 && width > 0, "row_norm_gate: %d rows of %d", rows, width);
    RI_REQUIRE(out_off >= 0 && out_off + width <= out_stride, "row_norm_gate: columns %d..+%d of rows of %d", out_off,
               width, out_stride);
    RI_REQUIRE(!gate || (g_off >= 0 && g_off + width <= gate_stride), "row_norm_gate: gates %d..+%d of rows of %d", g_off,
               width, gate_stride);
    RI_REQUIRE(kind == BR_GATE_SIGMOID || kind == BR_GATE_SILU, "row_norm_gate: gate kind %d", kind);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "row_norm_gate: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        row_norm_gate_kernel<float><<<rows, 256, 0, s>>>((float*)out + out_off, out_stride, x, gain, eps,
                                                         gate ? (const float*)gate + g_off : nullptr, gate_stride, scale, kind, width);
    else
        row_norm_gate_kernel<bf16_t><<<rows, 256, 0, s>>>((bf16_t*)out + out_off, out_stride, x, gain, eps,
                                                          gate ? (const bf16_t*)gate + g_off : nullptr, gate_stride, scale, kind, width);
    RI_LAUNCH_CHECK("row_norm_gate");
    return 0;
}
