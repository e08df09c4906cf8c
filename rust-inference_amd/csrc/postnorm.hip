// Row-wise kernels of layers whose norm sits behind the residual sum, and of their feed-forwards:
//   scaled_sum_norm:       r <- norm(alpha * r + y + y_bias): the residual itself is the norm's output (a layer norm with
//                          gain and bias, or an RMS norm with gain); y may come as parts of a split product, added in
//                          order, and y_bias is the bias of the product that made y; with a copy of the new r in the
//                          activations' format, which the next sublayer's products read;
//   glu_clamped_bias:      a = g sigmoid(1.702 g) (u + 1) with g = min(gate + b_gate, limit), u = clamp(up + b_up, -limit,
//                          limit), for rows [gate | up];
//   experts_activate_plain: a[t, e, :] = weight[t, e] * act(u[t, e, :]) for experts without a gate, zero for the experts a
//                          token did not choose;
//   softcap_rows:          x <- cap * tanh(x / cap) in place.
//
// The residual, the statistics, alpha and every activation are float32; a value is rounded once, when it is stored in
// the activations' format.  One workgroup a row; a row's sums are taken in an order that the row's width alone fixes.
#include "api.h"
#include "common.h"

#define PN_NORM_RMS 1
#define PN_NORM_LAYER 2

template <typename TY, typename TA>
__global__ void __launch_bounds__(256)
scaled_sum_norm_kernel(float* __restrict__ residual, TA* __restrict__ act, const TY* __restrict__ y, int parts,
                       size_t part_stride, const float* __restrict__ y_bias, float alpha, const float* __restrict__ gain,
                       const float* __restrict__ bias, float eps, int kind, int dim) {
    extern __shared__ float row[];                           // dim floats
    __shared__ float scratch[16];
    const size_t at = (size_t)blockIdx.x * dim;
    float sum = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = to_f32(y[at + d]);
        for (int p = 1; p < parts; ++p) v += to_f32(y[p * part_stride + at + d]);
        if (y_bias) v += y_bias[d];
        v += alpha * residual[at + d];
        row[d] = v;
        sum += v;
    }
    float mean = 0.f;
    if (kind == PN_NORM_LAYER) mean = block_sum(sum, scratch) / (float)dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float c = row[d] - mean;
        ss += c * c;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = (row[d] - mean) * inv * gain[d];
        if (bias) v += bias[d];
        residual[at + d] = v;
        if (act) from_f32(act + at + d, v);
    }
}

// 16 bytes of float32 or 8 of bfloat16 at once, as four floats.
__device__ __forceinline__ float4 pn_ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 pn_ld4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16),
                       __uint_as_float(w.y & 0xFFFF0000u));
}
__device__ __forceinline__ void pn_st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void pn_st4(bf16_t* p, float4 v) {
    uint2 w;
    w.x = pack_bf16x2(v.x, v.y);
    w.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = w;
}

// The same for rows of up to 1,024 * VPT elements, a multiple of 4: a thread asks for all its 16-byte pieces of the
// residual and of every part of y up front and keeps them in registers, so that a row is one trip to memory; the parts
// are added in their order, the row's sums taken in an order that the width alone fixes.
template <typename TY, typename TA, int VPT>
__global__ void __launch_bounds__(256)
scaled_sum_norm_vec_kernel(float* __restrict__ residual, TA* __restrict__ act, const TY* __restrict__ y, int parts,
                           size_t part_stride, const float* __restrict__ y_bias, float alpha, const float* __restrict__ gain,
                           const float* __restrict__ bias, float eps, int kind, int dim) {
    __shared__ float scratch[16];
    const size_t at = (size_t)blockIdx.x * dim;
    float4 v[VPT];
    int col[VPT];
    bool ok[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = (threadIdx.x + i * 256) * 4;
        ok[i] = c < dim;
        col[i] = ok[i] ? c : 0;                              // a column pulled back inside the row: the load is issued anyway
        const float4 r = pn_ld4(residual + at + col[i]);
        const float4 w = pn_ld4(y + at + col[i]);
        v[i] = make_float4(w.x, w.y, w.z, w.w);
        for (int p = 1; p < parts; ++p) {
            const float4 u = pn_ld4(y + p * part_stride + at + col[i]);
            v[i] = make_float4(v[i].x + u.x, v[i].y + u.y, v[i].z + u.z, v[i].w + u.w);
        }
        if (y_bias) {
            const float4 b = pn_ld4(y_bias + col[i]);
            v[i] = make_float4(v[i].x + b.x, v[i].y + b.y, v[i].z + b.z, v[i].w + b.w);
        }
        v[i] = make_float4(v[i].x + alpha * r.x, v[i].y + alpha * r.y, v[i].z + alpha * r.z, v[i].w + alpha * r.w);
    }
    float mean = 0.f;
    if (kind == PN_NORM_LAYER) {
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
        const float4 g = pn_ld4(gain + col[i]);
        float4 o = make_float4((v[i].x - mean) * inv * g.x, (v[i].y - mean) * inv * g.y, (v[i].z - mean) * inv * g.z,
                               (v[i].w - mean) * inv * g.w);
        if (bias) {
            const float4 b = pn_ld4(bias + col[i]);
            o = make_float4(o.x + b.x, o.y + b.y, o.z + b.z, o.w + b.w);
        }
        pn_st4(residual + at + col[i], o);
        if (act) pn_st4(act + at + col[i], o);
    }
}

extern "C" int ri_scaled_sum_norm(float* residual, void* act, int act_dtype, const void* y, int y_dtype, int parts,
                                  const float* y_bias, float alpha, const float* gain, const float* bias, float eps,
                                  int kind, int rows, int dim, void* stream) {
    RI_REQUIRE(rows > 0 && dim > 0 && parts >= 1, "scaled_sum_norm: %d rows of %d in %d parts", rows, dim, parts);
    RI_REQUIRE(kind == PN_NORM_RMS || kind == PN_NORM_LAYER, "scaled_sum_norm: norm kind %d", kind);
    RI_REQUIRE(gain && residual && y, "scaled_sum_norm: a gain, a residual and a branch output are needed");
    RI_REQUIRE((size_t)dim * sizeof(float) <= 64 * 1024, "scaled_sum_norm: rows of %d exceed the kernel's 16384", dim);
    RI_REQUIRE((y_dtype == RI_F32 || y_dtype == RI_BF16) && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "scaled_sum_norm: dtypes %d and %d", y_dtype, act_dtype);
    RI_REQUIRE(parts == 1 || y_dtype == RI_F32, "scaled_sum_norm: parts of a product are float32");
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)dim * sizeof(float), stride = (size_t)rows * dim;
#define RI_VEC(TY, TA, VPT)                                                                                             \
    scaled_sum_norm_vec_kernel<TY, TA, VPT><<<rows, 256, 0, s>>>(residual, (TA*)act, (const TY*)y, parts, stride, y_bias, \
                                                                 alpha, gain, bias, eps, kind, dim)
#define RI_GO(TY, TA)                                                                                                   \
    if (dim % 4 == 0 && dim <= 1024) RI_VEC(TY, TA, 1);                                                                 \
    else if (dim % 4 == 0 && dim <= 2048) RI_VEC(TY, TA, 2);                                                            \
    else if (dim % 4 == 0 && dim <= 4096) RI_VEC(TY, TA, 4);                                                            \
    else if (dim % 4 == 0 && dim <= 8192) RI_VEC(TY, TA, 8);                                                            \
    else                                                                                                                \
    scaled_sum_norm_kernel<TY, TA><<<rows, 256, lds, s>>>(residual, (TA*)act, (const TY*)y, parts, stride, y_bias, alpha, \
                                                          gain, bias, eps, kind, dim)
    if (y_dtype == RI_F32) { if (act_dtype == RI_F32) RI_GO(float, float); else RI_GO(float, bf16_t); }
    else                   { if (act_dtype == RI_F32) RI_GO(bf16_t, float); else RI_GO(bf16_t, bf16_t); }
#undef RI_GO
#undef RI_VEC
    RI_LAUNCH_CHECK("scaled_sum_norm");
    return 0;
}

// ------------------------------------------------------------------ the clamped gated activation with biases
template <typename T>
__global__ void __launch_bounds__(256)
glu_clamped_bias_kernel(T* __restrict__ out, const T* __restrict__ gu, const float* __restrict__ b_gate,
                        const float* __restrict__ b_up, float limit, int ff) {
    const size_t t = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= ff) return;
    float g = to_f32(gu[t * 2 * ff + i]), u = to_f32(gu[t * 2 * ff + ff + i]);
    if (b_gate) g += b_gate[i];
    if (b_up) u += b_up[i];
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    from_f32(out + t * ff + i, g / (1.f + expf(-1.702f * g)) * (u + 1.f));
}

// Rows whose width is a multiple of 8, in bfloat16: a thread takes eight neighbours of gate and of up in two 16-byte loads.
__global__ void __launch_bounds__(256)
glu_clamped_bias_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, const float* __restrict__ b_gate,
                               const float* __restrict__ b_up, float limit, int ff) {
    const size_t t = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= ff) return;
    const uint4 gq = *reinterpret_cast<const uint4*>(gu + t * 2 * ff + i);
    const uint4 uq = *reinterpret_cast<const uint4*>(gu + t * 2 * ff + ff + i);
    const uint32_t gw[4] = {gq.x, gq.y, gq.z, gq.w}, uw[4] = {uq.x, uq.y, uq.z, uq.w};
    float g[8], u[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        g[2 * e] = __uint_as_float(gw[e] << 16);
        g[2 * e + 1] = __uint_as_float(gw[e] & 0xFFFF0000u);
        u[2 * e] = __uint_as_float(uw[e] << 16);
        u[2 * e + 1] = __uint_as_float(uw[e] & 0xFFFF0000u);
    }
    float bg[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, bu[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (b_gate) {
        const float4 x = *reinterpret_cast<const float4*>(b_gate + i), y = *reinterpret_cast<const float4*>(b_gate + i + 4);
        bg[0] = x.x; bg[1] = x.y; bg[2] = x.z; bg[3] = x.w; bg[4] = y.x; bg[5] = y.y; bg[6] = y.z; bg[7] = y.w;
    }
    if (b_up) {
        const float4 x = *reinterpret_cast<const float4*>(b_up + i), y = *reinterpret_cast<const float4*>(b_up + i + 4);
        bu[0] = x.x; bu[1] = x.y; bu[2] = x.z; bu[3] = x.w; bu[4] = y.x; bu[5] = y.y; bu[6] = y.z; bu[7] = y.w;
    }
    uint32_t o[4];
    float a[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float gv = g[e] + bg[e], uv = u[e] + bu[e];
        gv = fminf(gv, limit);
        uv = fminf(fmaxf(uv, -limit), limit);
        a[e] = gv / (1.f + expf(-1.702f * gv)) * (uv + 1.f);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(a[2 * e], a[2 * e + 1]);
    *reinterpret_cast<uint4*>(out + t * ff + i) = make_uint4(o[0], o[1], o[2], o[3]);
}

extern "C" int ri_glu_clamped_bias(void* out, const void* gu, int dtype, const float* b_gate, const float* b_up,
                                   float limit, int rows, int ff, void* stream) {
    RI_REQUIRE(rows > 0, "glu_clamped_bias: %d rows", rows);
    RI_REQUIRE(ff > 0 && limit > 0.f, "glu_clamped_bias: width %d, limit %g", ff, (double)limit);
    RI_REQUIRE(dtype == RI_F32 || dtype == RI_BF16, "glu_clamped_bias: dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    for (int r0 = 0; r0 < rows; r0 += 65535) {                 // the grid's second axis takes 65,535 rows
        const int n = rows - r0 < 65535 ? rows - r0 : 65535;
        const dim3 grid((ff + 255) / 256, n);
        if (dtype == RI_F32)
            glu_clamped_bias_kernel<float><<<grid, 256, 0, s>>>((float*)out + (size_t)r0 * ff, (const float*)gu + (size_t)r0 * 2 * ff,
                                                               b_gate, b_up, limit, ff);
        else if (ff % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)b_gate % 16 == 0 &&
                 (uintptr_t)b_up % 16 == 0)
            glu_clamped_bias_bf16x8_kernel<<<dim3((ff / 8 + 255) / 256, n), 256, 0, s>>>(
                (bf16_t*)out + (size_t)r0 * ff, (const bf16_t*)gu + (size_t)r0 * 2 * ff, b_gate, b_up, limit, ff);
        else
            glu_clamped_bias_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out + (size_t)r0 * ff,
                                                                (const bf16_t*)gu + (size_t)r0 * 2 * ff, b_gate, b_up, limit, ff);
    }
    RI_LAUNCH_CHECK("glu_clamped_bias");
    return 0;
}

// ------------------------------------------------------------------ experts without a gate
#define PN_ACT_GELU_ERF 0
#define PN_ACT_GELU_TANH 1
#define PN_ACT_RELU2 2

__device__ __forceinline__ float pn_activate(float v, int kind) {
    if (kind == PN_ACT_GELU_ERF) return 0.5f * v * (1.f + erff(v * 0.7071067811865476f));
    if (kind == PN_ACT_GELU_TANH) return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    const float r = fmaxf(v, 0.f);
    return r * r;
}

template <typename T>
__global__ void __launch_bounds__(256)
experts_activate_plain_kernel(T* __restrict__ out, const T* __restrict__ u, const float* __restrict__ dense,
                              int dense_stride, int experts, int ff, int kind) {
    const size_t t = blockIdx.y;
    const int e = blockIdx.x;
    const float w = dense ? dense[t * dense_stride + e] : 1.f;
    const size_t at = (t * experts + e) * ff;
    for (int i = threadIdx.x; i < ff; i += 256)
        from_f32(out + at + i, w == 0.f ? 0.f : w * pn_activate(to_f32(u[at + i]), kind));
}

extern "C" int ri_experts_activate_plain(void* out, const void* u, int dtype, const float* dense, int dense_stride,
                                         int tokens, int experts, int ff, int kind, void* stream) {
    RI_REQUIRE(tokens > 0 && experts >= 1 && experts <= 65535 && ff >= 1, "experts_activate_plain: %d tokens, %d experts of %d",
               tokens, experts, ff);
    RI_REQUIRE(!dense || dense_stride >= experts, "experts_activate_plain: weight rows of %d for %d experts", dense_stride, experts);
    RI_REQUIRE(kind >= 0 && kind <= 2, "experts_activate_plain: activation %d", kind);
    RI_REQUIRE(dtype == RI_F32 || dtype == RI_BF16, "experts_activate_plain: dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    for (int r0 = 0; r0 < tokens; r0 += 65535) {
        const int n = tokens - r0 < 65535 ? tokens - r0 : 65535;
        const dim3 grid(experts, n);
        const size_t at = (size_t)r0 * experts * ff;
        const float* d = dense ? dense + (size_t)r0 * dense_stride : nullptr;
        if (dtype == RI_F32)
            experts_activate_plain_kernel<float><<<grid, 256, 0, s>>>((float*)out + at, (const float*)u + at, d, dense_stride,
                                                                     experts, ff, kind);
        else
            experts_activate_plain_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out + at, (const bf16_t*)u + at, d, dense_stride,
                                                                      experts, ff, kind);
    }
    RI_LAUNCH_CHECK("experts_activate_plain");
    return 0;
}

// ------------------------------------------------------------------ a cap on the logits
__global__ void softcap_kernel(float* __restrict__ x, float cap, long total) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < total) x[e] = cap * tanhf(x[e] / cap);
}

extern "C" int ri_softcap_rows(float* x, float cap, long total, void* stream) {
    RI_REQUIRE(total > 0 && cap > 0.f, "softcap_rows: %ld elements, cap %g", total, (double)cap);
    RI_REQUIRE((total + 255) / 256 <= 2147483647L, "softcap_rows: %ld elements exceed one launch", total);
    softcap_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, cap, total);
    RI_LAUNCH_CHECK("softcap_rows");
    return 0;
}
