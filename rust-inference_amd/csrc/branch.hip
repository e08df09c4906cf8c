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

// 16 bytes of float32 or 8 of bfloat16 at once, as four floats.
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16),
                       __uint_as_float(w.y & 0xFFFF0000u));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
    uint2 w;
    w.x = pack_bf16x2(v.x, v.y);
    w.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = w;
}

// Rows whose width is a multiple of 4: a thread takes four neighbours, a workgroup 1,024 columns of one row.
template <typename TW, typename TA>
__global__ void __launch_bounds__(256)
embed_scaled_vec_kernel(float* __restrict__ out, TA* __restrict__ act, const TW* __restrict__ table,
                        const int32_t* __restrict__ ids, float scale, int dim) {
    const int t = blockIdx.x, c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c >= dim) return;
    float4 v = ld4(table + (size_t)ids[t] * dim + c);
    v = make_float4(v.x * scale, v.y * scale, v.z * scale, v.w * scale);
    st4(out + (size_t)t * dim + c, v);
    if (act) st4(act + (size_t)t * dim + c, v);
}

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
    const dim3 vgrid(tokens, (dim / 4 + 255) / 256);
#define RI_GO(TW, TA)                                                                                                   \
    if (dim % 4 == 0 && vgrid.y <= 65535)                                                                               \
        embed_scaled_vec_kernel<TW, TA><<<vgrid, 256, 0, s>>>(out, (TA*)act, (const TW*)table, ids, scale, dim);        \
    else                                                                                                                \
        embed_scaled_kernel<TW, TA><<<tokens, 256, 0, s>>>(out, (TA*)act, (const TW*)table, ids, scale, dim)
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

// The same for rows of up to 8,192 elements, a multiple of 4: a thread asks for all its 16-byte pieces of the residual
// and of every part of y up front and keeps them in registers, so that a row is one trip to memory and not one an
// element; the parts are added in their order, the row's sums taken in an order that the width alone fixes.
template <typename TY, typename TA, int VPT>
__global__ void __launch_bounds__(256)
branch_norm_add_vec_kernel(float* __restrict__ residual, TA* __restrict__ act, const TY* __restrict__ y, int parts,
                           size_t part_stride, const float* __restrict__ gain, const float* __restrict__ bias, float eps,
                           int kind, const float* __restrict__ layer_scale, int dim) {
    __shared__ float scratch[16];
    const size_t at = (size_t)blockIdx.x * dim;
    float4 r[VPT], v[VPT];
    int col[VPT];
    bool ok[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = (threadIdx.x + i * 256) * 4;
        ok[i] = c < dim;
        col[i] = ok[i] ? c : 0;                              // a column pulled back inside the row: the load is issued anyway
        r[i] = ld4(residual + at + col[i]);
        v[i] = ld4(y + at + col[i]);
    }
    for (int p = 1; p < parts; ++p) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const float4 w = ld4(y + p * part_stride + at + col[i]);
            v[i] = make_float4(v[i].x + w.x, v[i].y + w.y, v[i].z + w.z, v[i].w + w.w);
        }
    }
    float mean = 0.f;
    if (kind == BR_NORM_LAYER) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < VPT; ++i)
            if (ok[i]) sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
        mean = block_sum(sum, scratch) / (float)dim;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (ok[i]) {
            const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
            ss += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (!ok[i]) continue;
        const float4 g = ld4(gain + col[i]);
        float4 o = make_float4((v[i].x - mean) * inv * g.x, (v[i].y - mean) * inv * g.y, (v[i].z - mean) * inv * g.z,
                               (v[i].w - mean) * inv * g.w);
        if (bias) {
            const float4 b = ld4(bias + col[i]);
            o = make_float4(o.x + b.x, o.y + b.y, o.z + b.z, o.w + b.w);
        }
        if (layer_scale) {
            const float4 l = ld4(layer_scale + col[i]);
            o = make_float4(o.x * l.x, o.y * l.y, o.z * l.z, o.w * l.w);
        }
        o = make_float4(r[i].x + o.x, r[i].y + o.y, r[i].z + o.z, r[i].w + o.w);
        st4(residual + at + col[i], o);
        if (act) st4(act + at + col[i], o);
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
#define RI_VEC(TY, TA, VPT)                                                                                             \
    branch_norm_add_vec_kernel<TY, TA, VPT><<<rows, 256, 0, s>>>(residual, (TA*)act, (const TY*)y, parts, stride, gain,   \
                                                                 bias, eps, kind, layer_scale, dim)
#define RI_GO(TY, TA)                                                                                                   \
    if (dim % 4 == 0 && dim <= 1024) RI_VEC(TY, TA, 1);                                                                 \
    else if (dim % 4 == 0 && dim <= 2048) RI_VEC(TY, TA, 2);                                                            \
    else if (dim % 4 == 0 && dim <= 4096) RI_VEC(TY, TA, 4);                                                            \
    else if (dim % 4 == 0 && dim <= 8192) RI_VEC(TY, TA, 8);                                                            \
    else                                                                                                                \
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
#undef RI_VEC
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

// Widths, offsets and row lengths that are multiples of 4: a thread takes four neighbours, a workgroup 1,024 columns.
template <typename TX, typename TA>
__global__ void __launch_bounds__(256)
gate_rows_vec_kernel(TA* __restrict__ out, int out_stride, const TX* __restrict__ x, const TA* __restrict__ gate,
                     int gate_stride, float scale, int kind, int width) {
    const size_t t = blockIdx.x;
    const int d = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (d >= width) return;
    float4 v = ld4(x + t * width + d);
    v = make_float4(v.x * scale, v.y * scale, v.z * scale, v.w * scale);
    if (gate) {
        const float4 g = ld4(gate + t * gate_stride + d);
        v = make_float4(v.x * gate_of(g.x, kind), v.y * gate_of(g.y, kind), v.z * gate_of(g.z, kind), v.w * gate_of(g.w, kind));
    }
    st4(out + t * out_stride + d, v);
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
    const bool vec = (width | out_off | out_stride) % 4 == 0 && (!gate || (g_off | gate_stride) % 4 == 0) &&
                     (width / 4 + 255) / 256 <= 65535;
    const dim3 vgrid(rows, (width / 4 + 255) / 256);
#define RI_GO(TX, TA)                                                                                                  \
    if (vec)                                                                                                           \
        gate_rows_vec_kernel<TX, TA><<<vgrid, 256, 0, s>>>((TA*)out + out_off, out_stride, (const TX*)x,                  \
                                                           gate ? (const TA*)gate + g_off : nullptr, gate_stride, scale, \
                                                           kind, width);                                                \
    else                                                                                                               \
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

// Rows of up to 8,192 elements whose width, offsets and row lengths are multiples of 4: a row in registers, one trip.
template <typename TA, int VPT>
__global__ void __launch_bounds__(256)
row_norm_gate_vec_kernel(TA* __restrict__ out, int out_stride, const float* __restrict__ x, const float* __restrict__ gain,
                         float eps, const TA* __restrict__ gate, int gate_stride, float scale, int kind, int width) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    float4 v[VPT], g[VPT];
    int col[VPT];
    bool ok[VPT];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = (threadIdx.x + i * 256) * 4;
        ok[i] = c < width;
        col[i] = ok[i] ? c : 0;
        v[i] = ld4(x + t * width + col[i]);
        g[i] = gate ? ld4(gate + t * gate_stride + col[i]) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i)
        if (ok[i]) ss += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    const float f = scale / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        if (!ok[i]) continue;
        float4 o = make_float4(v[i].x * f, v[i].y * f, v[i].z * f, v[i].w * f);
        if (gain) {
            const float4 w = ld4(gain + col[i]);
            o = make_float4(o.x * w.x, o.y * w.y, o.z * w.z, o.w * w.w);
        }
        if (gate)
            o = make_float4(o.x * gate_of(g[i].x, kind), o.y * gate_of(g[i].y, kind), o.z * gate_of(g[i].z, kind),
                            o.w * gate_of(g[i].w, kind));
        st4(out + t * out_stride + col[i], o);
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
    if ((width | out_off | out_stride) % 4 == 0 && (!gate || (g_off | gate_stride) % 4 == 0) && width <= 8192) {
#define RI_VEC(TA, VPT)                                                                                                 \
    row_norm_gate_vec_kernel<TA, VPT><<<rows, 256, 0, s>>>((TA*)out + out_off, out_stride, x, gain, eps,                   \
                                                           gate ? (const TA*)gate + g_off : nullptr, gate_stride, scale,  \
                                                           kind, width)
#define RI_GO(TA)                                                                                                       \
    if (width <= 1024) RI_VEC(TA, 1); else if (width <= 2048) RI_VEC(TA, 2); else if (width <= 4096) RI_VEC(TA, 4);       \
    else RI_VEC(TA, 8)
        if (act_dtype == RI_F32) { RI_GO(float); } else { RI_GO(bf16_t); }
#undef RI_GO
#undef RI_VEC
        RI_LAUNCH_CHECK("row_norm_gate");
        return 0;
    }
    if (act_dtype == RI_F32)
        row_norm_gate_kernel<float><<<rows, 256, 0, s>>>((float*)out + out_off, out_stride, x, gain, eps,
                                                         gate ? (const float*)gate + g_off : nullptr, gate_stride, scale, kind, width);
    else
        row_norm_gate_kernel<bf16_t><<<rows, 256, 0, s>>>((bf16_t*)out + out_off, out_stride, x, gain, eps,
                                                          gate ? (const bf16_t*)gate + g_off : nullptr, gate_stride, scale, kind, width);
    RI_LAUNCH_CHECK("row_norm_gate");
    return 0;
}
