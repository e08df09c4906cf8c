// Queries and keys made ready for an attention without rotation, and keys and values into their pages, in one
// pass over the fused projection [tokens][heads * dim | kv_heads * dim | kv_heads * vdim] (the value heads may
// have another size than the query and key heads).
//
//   q, k: optional per-head RMS norm, x / sqrt(mean(x^2) + eps) * gain, one gain of `dim` for all heads;
//   q:    a temperature by position, q *= 1 + coef * ln(floor((p + 1) / every) + 1) (coef 0: none), in place;
//   k:    into k_pages [pages][kv_heads][page_size][dim];
//   v:    copied into v_pages [pages][kv_heads][vdim][page_size] (transposed inside a page).
//
// Norm, logarithm and factor are float32; a q or k element is rounded once.  One wavefront per (token, head) in
// the general kernel; prompts of head sizes that allow it go through the 16-byte kernels further down.
#include "api.h"
#include "common.h"

#define QT_MAX_PER_LANE 8    // head sizes up to 64 * 8

template <typename TA, typename TC>
__global__ void qk_norm_temper_kv_write_kernel(
    TA* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    float temp_coef, int temp_every, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ page_table, int table_width, TC* __restrict__ k_pages, TC* __restrict__ v_pages,
    int tokens, int heads, int kv_heads, int dim, int vdim, int page_size) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int all_heads = heads + 2 * kv_heads;
    const long item = (long)blockIdx.x * (blockDim.x / RI_WAVE) + threadIdx.x / RI_WAVE;
    if (item >= (long)tokens * all_heads) return;          // whole wavefront leaves together
    const int t = (int)(item / all_heads), hh = (int)(item % all_heads);
    const size_t row_len = (size_t)(heads + kv_heads) * dim + (size_t)kv_heads * vdim;
    TA* row = qkv + (size_t)t * row_len;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    if (hh >= heads + kv_heads) {
        const int kvh = hh - heads - kv_heads;
        const TA* x = row + (size_t)(heads + kv_heads) * dim + (size_t)kvh * vdim;
        TC* vt = v_pages + ((size_t)page * kv_heads + kvh) * page_size * vdim + pos % page_size;
        for (int d = lane; d < vdim; d += RI_WAVE) from_f32(vt + (size_t)d * page_size, to_f32(x[d]));
        return;
    }
    TA* x = row + (size_t)hh * dim;
    float v[QT_MAX_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QT_MAX_PER_LANE; ++j) {
        const int i = lane + j * RI_WAVE;
        v[j] = i < dim ? to_f32(x[i]) : 0.f;
        ss += v[j] * v[j];
    }
    const bool is_q = hh < heads;
    const float* gain = is_q ? q_gain : k_gain;
    float f = 1.0f;
    if (gain) f = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
    float temper = 1.0f;
    if (is_q && temp_coef != 0.f) temper = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
    TC* dst = is_q ? nullptr
                   : k_pages + (((size_t)page * kv_heads + (hh - heads)) * page_size + pos % page_size) * dim;
#pragma unroll
    for (int j = 0; j < QT_MAX_PER_LANE; ++j) {
        const int i = lane + j * RI_WAVE;
        if (i >= dim) continue;
        float a = v[j];
        if (gain) a = a * f * gain[i];
        if (is_q) from_f32(x + i, a * temper);
        else      from_f32(dst + i, a);
    }
}

// ------------------------------------------------------------------ prompts: 16 bytes a lane, values a page at a time
// For steps with more than one new token a sequence and head sizes of 8 lanes' worth of eight elements or a
// power-of-two fraction (dim 8, 16, ... 512): a lane takes eight consecutive elements of a q or k head, so dim / 8
// lanes make a head and a wavefront works on 512 / dim heads at once, every load and store 16 bytes (32 for
// float32); one workgroup a token.  Values are written by the page-wise kernel below.
template <typename T> struct Eight;
template <> struct Eight<float> {
    __device__ static void load(const float* p, float* o) {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
    __device__ static void store(float* p, const float* v) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};
template <> struct Eight<bf16_t> {
    __device__ static void load(const bf16_t* p, float* o) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = __uint_as_float(w[i] << 16);
            o[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        }
    }
    __device__ static void store(bf16_t* p, const float* v) {
        *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                                                  pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
    }
};

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
qk_norm_temper_k_write_vec_kernel(TA* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain,
                                  float eps, float temp_coef, int temp_every, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table,
                                  int table_width, TC* __restrict__ k_pages, int heads, int kv_heads, int dim, int vdim,
                                  int page_size) {
    const int lane = threadIdx.x & (RI_WAVE - 1), wave = threadIdx.x / RI_WAVE;
    const int t = blockIdx.x;
    const int lanes_per_head = dim / 8;                      // a power of two, at most 64
    const int heads_at_once = RI_WAVE / lanes_per_head;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    const float temper = temp_coef != 0.f ? 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f) : 1.0f;
    const int qk_heads = heads + kv_heads;
    TA* row = qkv + (size_t)t * ((size_t)qk_heads * dim + (size_t)kv_heads * vdim);
    const int sub = lane / lanes_per_head, piece = lane % lanes_per_head;
    for (int h0 = wave * heads_at_once; h0 < qk_heads; h0 += 4 * heads_at_once) {
        const int hh = h0 + sub;
        if (hh >= qk_heads) continue;                        // lanes of a head stay together: the shuffles below are safe
        TA* x = row + (size_t)hh * dim + piece * 8;
        float a[8];
        Eight<TA>::load(x, a);
        const bool is_q = hh < heads;
        const float* gain = is_q ? q_gain : k_gain;
        if (gain) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += a[e] * a[e];
            for (int m = lanes_per_head / 2; m > 0; m >>= 1) ss += __shfl_xor(ss, m, RI_WAVE);
            const float f = 1.0f / sqrtf(ss / (float)dim + eps);
            float g[8];
            Eight<float>::load(gain + piece * 8, g);
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = a[e] * f * g[e];
        }
        if (is_q) {
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] *= temper;
            Eight<TA>::store(x, a);
        } else {
            Eight<TC>::store(k_pages + (((size_t)page * kv_heads + (hh - heads)) * page_size + pos % page_size) * dim + piece * 8, a);
        }
    }
}

// Values into their pages, a page at a time: one workgroup per (32 positions touched by this step, sequence, kv
// head) reads the new tokens' value heads as rows, turns them through LDS and writes channel rows.
#define QT_TOKENS 32
template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
values_to_pages_kernel(const TA* __restrict__ qkv, size_t row_len, size_t v_off, const int32_t* __restrict__ cu_seqlens,
                       const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                       TC* __restrict__ v_pages, int kv_heads, int vdim, int page_size) {
    extern __shared__ float tile[];                          // [QT_TOKENS][vdim + 1]
    const int b = blockIdx.y, kvh = blockIdx.z;
    const int t_begin = cu_seqlens[b], n = cu_seqlens[b + 1] - t_begin;
    if (n <= 0) return;
    const int start = tok_pos[t_begin];                      // the sequence's new tokens sit at start .. start + n - 1
    const int first = (start / QT_TOKENS + blockIdx.x) * QT_TOKENS;
    const int lo = max(first, start), hi = min(first + QT_TOKENS - 1, start + n - 1);
    if (lo > hi) return;
    const int stride = vdim + 1;
    const TA* from = qkv + v_off + (size_t)kvh * vdim;
    const bool whole = lo == first && hi == first + QT_TOKENS - 1;
    if (sizeof(TA) == 2 && whole && vdim % 8 == 0 && (row_len % 8) == 0 && (v_off % 8) == 0) {
        const int pieces = vdim / 8;
        for (int e = threadIdx.x; e < QT_TOKENS * pieces; e += blockDim.x) {
            const int tt = e / pieces, d = (e - tt * pieces) * 8;
            float v[8];
            Eight<TA>::load(from + (size_t)(t_begin + first - start + tt) * row_len + d, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) tile[tt * stride + d + j] = v[j];
        }
    } else {
        for (int e = threadIdx.x; e < (hi - lo + 1) * vdim; e += blockDim.x) {
            const int tt = e / vdim, d = e - tt * vdim;
            tile[(lo - first + tt) * stride + d] = to_f32(from[(size_t)(t_begin + lo - start + tt) * row_len + d]);
        }
    }
    __syncthreads();
    const int page = page_table[(size_t)b * table_width + first / page_size];
    TC* base = v_pages + ((size_t)page * kv_heads + kvh) * page_size * vdim + first % page_size;
    if (whole && page_size % 8 == 0) {
        for (int e = threadIdx.x; e < vdim * (QT_TOKENS / 8); e += blockDim.x) {
            const int d = e / (QT_TOKENS / 8), t8 = (e - d * (QT_TOKENS / 8)) * 8;
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = tile[(t8 + j) * stride + d];
            Eight<TC>::store(base + (size_t)d * page_size + t8, v);
        }
    } else {
        for (int e = threadIdx.x; e < vdim * QT_TOKENS; e += blockDim.x) {
            const int d = e / QT_TOKENS, tt = e - d * QT_TOKENS;
            if (first + tt >= lo && first + tt <= hi) from_f32(base + (size_t)d * page_size + tt, tile[tt * stride + d]);
        }
    }
}

template <typename TA, typename TC>
static void launch_qk_temper(void* qkv, const float* q_gain, const float* k_gain, float eps, float temp_coef, int temp_every,
                             const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* cu_seqlens, int seqs, int max_new,
                             const int32_t* page_table, int table_width, void* k_pages, void* v_pages, int tokens,
                             int heads, int kv_heads, int dim, int vdim, int page_size, hipStream_t s) {
    const int lph = dim / 8;
    const size_t row_len = (size_t)(heads + kv_heads) * dim + (size_t)kv_heads * vdim;
    const bool pieces_fit = dim % 8 == 0 && lph <= 64 && (lph & (lph - 1)) == 0 &&
                            (sizeof(TA) == 2 ? (row_len % 8 == 0) : (row_len % 4 == 0));
    if (cu_seqlens && max_new > 1 && pieces_fit && page_size % QT_TOKENS == 0 && seqs <= 65535 && kv_heads <= 65535 &&
        (size_t)QT_TOKENS * (vdim + 1) * sizeof(float) <= 65536) {
        qk_norm_temper_k_write_vec_kernel<TA, TC><<<tokens, 256, 0, s>>>(
            (TA*)qkv, q_gain, k_gain, eps, temp_coef, temp_every, tok_pos, tok_seq, page_table, table_width, (TC*)k_pages,
            heads, kv_heads, dim, vdim, page_size);
        dim3 grid((max_new + QT_TOKENS - 2) / QT_TOKENS + 1, seqs, kv_heads);      // the 32-position pieces a sequence may touch
        values_to_pages_kernel<TA, TC><<<grid, 256, QT_TOKENS * (vdim + 1) * sizeof(float), s>>>(
            (const TA*)qkv, row_len, (size_t)(heads + kv_heads) * dim, cu_seqlens, tok_pos, page_table, table_width,
            (TC*)v_pages, kv_heads, vdim, page_size);
        return;
    }
    const long items = (long)tokens * (heads + 2 * kv_heads);
    qk_norm_temper_kv_write_kernel<TA, TC><<<(unsigned)((items + 3) / 4), 256, 0, s>>>(
        (TA*)qkv, q_gain, k_gain, eps, temp_coef, temp_every, tok_pos, tok_seq, page_table, table_width, (TC*)k_pages,
        (TC*)v_pages, tokens, heads, kv_heads, dim, vdim, page_size);
}

extern "C" int ri_qk_norm_temper_kv_write(void* qkv, int act_dtype, const float* q_gain, const float* k_gain, float eps,
                                          float temp_coef, int temp_every, const int32_t* tok_pos,
                                          const int32_t* tok_seq, const int32_t* cu_seqlens, int seqs, int max_new,
                                          const int32_t* page_table, int table_width,
                                          void* k_pages, void* v_pages, int cache_dtype, int tokens, int heads,
                                          int kv_heads, int dim, int vdim, int page_size, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0, "qk_norm_temper_kv_write: tokens %d, heads %d, kv heads %d", tokens,
               heads, kv_heads);
    RI_REQUIRE(dim >= 1 && dim <= RI_WAVE * QT_MAX_PER_LANE && vdim >= 1, "qk_norm_temper_kv_write: head sizes %d and %d",
               dim, vdim);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "qk_norm_temper_kv_write: activations (%d) and cache (%d) must share float32 or bfloat16", act_dtype,
               cache_dtype);
    RI_REQUIRE(temp_coef == 0.f || temp_every >= 1, "qk_norm_temper_kv_write: a temperature every %d positions", temp_every);
    RI_REQUIRE(page_size > 0 && table_width > 0 && k_pages && v_pages, "qk_norm_temper_kv_write: page geometry");
    const long items = (long)tokens * (heads + 2 * kv_heads);
    const long blocks = (items + 3) / 4;
    RI_REQUIRE(blocks <= 2147483647L, "qk_norm_temper_kv_write: %ld heads exceed one launch", items);
    RI_REQUIRE(!cu_seqlens || (seqs > 0 && max_new > 0), "qk_norm_temper_kv_write: seqs %d, max_new %d", seqs, max_new);
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        launch_qk_temper<float, float>(qkv, q_gain, k_gain, eps, temp_coef, temp_every, tok_pos, tok_seq, cu_seqlens, seqs,
                                       max_new, page_table, table_width, k_pages, v_pages, tokens, heads, kv_heads, dim,
                                       vdim, page_size, s);
    else
        launch_qk_temper<bf16_t, bf16_t>(qkv, q_gain, k_gain, eps, temp_coef, temp_every, tok_pos, tok_seq, cu_seqlens,
                                         seqs, max_new, page_table, table_width, k_pages, v_pages, tokens, heads,
                                         kv_heads, dim, vdim, page_size, s);
    RI_LAUNCH_CHECK("qk_norm_temper_kv_write");
    return 0;
}

// ------------------------------------------------------------------ rotation of neighbours, then the norm
// Queries and keys of an attention whose rotation turns the neighbours (2i, 2i + 1) of the first rot_dims elements
// of every head by pos * inv_freq[i] (the rest of the head passes), followed by a per-head RMS norm (with a gain of
// `dim`, or without one: unit_norm), from a projection row that may hold more than this mixer's columns: q heads
// at q_off, k heads at k_off, v heads at v_off of rows of row_len elements.  q in place, k and v into their pages.
// Angle, sine and cosine, and the norm are float32; an element is rounded once.  One wavefront per (token, head),
// a lane on pairs of neighbours; a prompt's values go a page at a time (values_to_pages_kernel).
#define QP_PAIRS_PER_LANE 4     // head sizes up to 64 * 2 * 4

// HPW: heads a wavefront takes one after the other (all of one token, so that the angles' sines and cosines are made
// once for them, and their loads are in flight together); a prompt runs with 4, single tokens with 1.
template <typename TA, typename TC, int HPW>
__global__ void qk_pairs_norm_kv_write_kernel(
    TA* __restrict__ proj, size_t row_len, int q_off, int k_off, int v_off, const float* __restrict__ inv_freq,
    int rot_dims, const float* __restrict__ q_gain, const float* __restrict__ k_gain, int norm, float eps,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table,
    int table_width, TC* __restrict__ k_pages, TC* __restrict__ v_pages, int tokens, int heads, int kv_heads, int dim,
    int vdim, int page_size, int write_values) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const int all_heads = heads + (write_values ? 2 : 1) * kv_heads;   // without the values, only q and k heads are items
    const int runs = (all_heads + HPW - 1) / HPW;                      // a token's heads in runs of HPW
    const long item = (long)blockIdx.x * (blockDim.x / RI_WAVE) + threadIdx.x / RI_WAVE;
    if (item >= (long)tokens * runs) return;               // whole wavefront leaves together
    const int t = (int)(item / runs), h0 = (int)(item % runs) * HPW;
    TA* row = proj + (size_t)t * row_len;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    float a[HPW][QP_PAIRS_PER_LANE], b[HPW][QP_PAIRS_PER_LANE];
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
        const int hh = h0 + u;
        if (hh >= heads + kv_heads) continue;               // a value head, or none: below
        const TA* x = row + (hh < heads ? q_off + (size_t)hh * dim : k_off + (size_t)(hh - heads) * dim);
#pragma unroll
        for (int j = 0; j < QP_PAIRS_PER_LANE; ++j) {
            const int i = 2 * (lane + j * RI_WAVE);          // this pair: elements i and i + 1
            a[u][j] = i < dim ? to_f32(x[i]) : 0.f;
            b[u][j] = i + 1 < dim ? to_f32(x[i + 1]) : 0.f;
        }
    }
    float sn[QP_PAIRS_PER_LANE], cs[QP_PAIRS_PER_LANE];
#pragma unroll
    for (int j = 0; j < QP_PAIRS_PER_LANE; ++j) {
        const int i = 2 * (lane + j * RI_WAVE);
        sn[j] = 0.f;
        cs[j] = 1.f;
        if (i + 1 < rot_dims) sincosf((float)pos * inv_freq[i / 2], &sn[j], &cs[j]);
    }
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
        const int hh = h0 + u;
        if (hh >= all_heads) continue;
        if (hh >= heads + kv_heads) {                        // a value head: copied into its page, transposed
            const int kvh = hh - heads - kv_heads;
            const TA* x = row + v_off + (size_t)kvh * vdim;
            TC* vt = v_pages + ((size_t)page * kv_heads + kvh) * page_size * vdim + pos % page_size;
            for (int d = lane; d < vdim; d += RI_WAVE) from_f32(vt + (size_t)d * page_size, to_f32(x[d]));
            continue;
        }
        const bool is_q = hh < heads;
        TA* x = row + (is_q ? q_off + (size_t)hh * dim : k_off + (size_t)(hh - heads) * dim);
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < QP_PAIRS_PER_LANE; ++j) {
            const int i = 2 * (lane + j * RI_WAVE);
            if (i + 1 < rot_dims) {
                const float p = a[u][j], q = b[u][j];
                a[u][j] = p * cs[j] - q * sn[j];
                b[u][j] = q * cs[j] + p * sn[j];
            }
            ss += a[u][j] * a[u][j] + b[u][j] * b[u][j];
        }
        const float* gain = is_q ? q_gain : k_gain;
        const float f = norm ? 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps) : 1.0f;
        TC* dst = is_q ? nullptr
                       : k_pages + (((size_t)page * kv_heads + (hh - heads)) * page_size + pos % page_size) * dim;
#pragma unroll
        for (int j = 0; j < QP_PAIRS_PER_LANE; ++j) {
            const int i = 2 * (lane + j * RI_WAVE);
            if (i < dim) {
                const float v = a[u][j] * f * (gain ? gain[i] : 1.0f);
                if (is_q) from_f32(x + i, v); else from_f32(dst + i, v);
            }
            if (i + 1 < dim) {
                const float v = b[u][j] * f * (gain ? gain[i + 1] : 1.0f);
                if (is_q) from_f32(x + i + 1, v); else from_f32(dst + i + 1, v);
            }
        }
    }
}

// A prompt with head sizes that 16-byte pieces divide (8 times a power of two, up to 512): a workgroup a token, a lane
// on eight neighbours (four pairs) of a head, so that a wavefront takes 512 / dim heads at once; the four angles'
// sines and cosines are made once a lane and serve every head of the token.  q in place, k into its page; the values
// go a page at a time (values_to_pages_kernel).
template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
qk_pairs_norm_k_write_vec_kernel(TA* __restrict__ proj, size_t row_len, int q_off, int k_off,
                                 const float* __restrict__ inv_freq, int rot_dims, const float* __restrict__ q_gain,
                                 const float* __restrict__ k_gain, int norm, float eps, const int32_t* __restrict__ tok_pos,
                                 const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width,
                                 TC* __restrict__ k_pages, int heads, int kv_heads, int dim, int page_size) {
    const int lane = threadIdx.x & (RI_WAVE - 1), wave = threadIdx.x / RI_WAVE;
    const int t = blockIdx.x;
    const int lanes_per_head = dim / 8;                      // a power of two, at most 64
    const int heads_at_once = RI_WAVE / lanes_per_head;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    const int qk_heads = heads + kv_heads;
    TA* row = proj + (size_t)t * row_len;
    const int sub = lane / lanes_per_head, piece = lane % lanes_per_head;
    float sn[4], cs[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int i = piece * 8 + 2 * e;                     // this pair: elements i and i + 1 of a head
        sn[e] = 0.f;
        cs[e] = 1.f;
        if (i + 1 < rot_dims) sincosf((float)pos * inv_freq[i / 2], &sn[e], &cs[e]);
    }
    for (int h0 = wave * heads_at_once; h0 < qk_heads; h0 += 4 * heads_at_once) {
        const int hh = h0 + sub;
        if (hh >= qk_heads) continue;                        // lanes of a head stay together: the shuffles below are safe
        const bool is_q = hh < heads;
        TA* x = row + (is_q ? q_off + (size_t)hh * dim : k_off + (size_t)(hh - heads) * dim) + piece * 8;
        float a[8];
        Eight<TA>::load(x, a);
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float u = a[2 * e], v = a[2 * e + 1];
            a[2 * e] = u * cs[e] - v * sn[e];
            a[2 * e + 1] = v * cs[e] + u * sn[e];
            ss += a[2 * e] * a[2 * e] + a[2 * e + 1] * a[2 * e + 1];
        }
        if (norm) {
            for (int m = lanes_per_head / 2; m > 0; m >>= 1) ss += __shfl_xor(ss, m, RI_WAVE);
            const float f = 1.0f / sqrtf(ss / (float)dim + eps);
            const float* gain = is_q ? q_gain : k_gain;
            float g[8];
            if (gain) Eight<float>::load(gain + piece * 8, g);
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = a[e] * f * (gain ? g[e] : 1.0f);
        }
        if (is_q) Eight<TA>::store(x, a);
        else Eight<TC>::store(k_pages + (((size_t)page * kv_heads + (hh - heads)) * page_size + pos % page_size) * dim + piece * 8, a);
    }
}

extern "C" int ri_qk_pairs_norm_kv_write(void* proj, int act_dtype, long row_len, int q_off, int k_off, int v_off,
                                         const float* inv_freq, int rot_dims, const float* q_gain, const float* k_gain,
                                         int norm, float eps, const int32_t* tok_pos, const int32_t* tok_seq,
                                         const int32_t* cu_seqlens, int seqs, int max_new, const int32_t* page_table,
                                         int table_width, void* k_pages, void* v_pages, int cache_dtype, int tokens,
                                         int heads, int kv_heads, int dim, int vdim, int page_size, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0, "qk_pairs_norm_kv_write: tokens %d, heads %d, kv heads %d", tokens,
               heads, kv_heads);
    RI_REQUIRE(dim >= 1 && dim <= RI_WAVE * 2 * QP_PAIRS_PER_LANE && vdim >= 1, "qk_pairs_norm_kv_write: head sizes %d and %d",
               dim, vdim);
    RI_REQUIRE(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq),
               "qk_pairs_norm_kv_write: a rotation over %d of %d elements", rot_dims, dim);
    RI_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + (long)heads * dim <= row_len &&
               k_off + (long)kv_heads * dim <= row_len && v_off + (long)kv_heads * vdim <= row_len,
               "qk_pairs_norm_kv_write: q, k, v at %d, %d, %d do not fit rows of %ld", q_off, k_off, v_off, row_len);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "qk_pairs_norm_kv_write: activations (%d) and cache (%d) must share float32 or bfloat16", act_dtype, cache_dtype);
    RI_REQUIRE(page_size > 0 && table_width > 0 && k_pages && v_pages, "qk_pairs_norm_kv_write: page geometry");
    RI_REQUIRE((!q_gain && !k_gain) || norm, "qk_pairs_norm_kv_write: gains without a norm");
    RI_REQUIRE(((long)tokens * (heads + 2 * kv_heads) + 3) / 4 <= 2147483647L, "qk_pairs_norm_kv_write: %ld heads exceed one launch",
               (long)tokens * (heads + 2 * kv_heads));
    RI_REQUIRE(!cu_seqlens || (seqs > 0 && max_new > 0), "qk_pairs_norm_kv_write: seqs %d, max_new %d", seqs, max_new);
    hipStream_t s = (hipStream_t)stream;
    // a prompt's values a page at a time, where the sizes allow it
    const bool paged_values = cu_seqlens && max_new > 1 && page_size % QT_TOKENS == 0 && seqs <= 65535 && kv_heads <= 65535 &&
                              (size_t)QT_TOKENS * (vdim + 1) * sizeof(float) <= 65536;
    const int lph = dim / 8, unit = act_dtype == RI_BF16 ? 8 : 4;
    if (paged_values && dim % 8 == 0 && lph <= 64 && (lph & (lph - 1)) == 0 && row_len % unit == 0 && q_off % unit == 0 &&
        k_off % unit == 0) {
#define RI_VEC(T)                                                                                                       \
    qk_pairs_norm_k_write_vec_kernel<T, T><<<tokens, 256, 0, s>>>(                                                        \
        (T*)proj, (size_t)row_len, q_off, k_off, inv_freq, rot_dims, q_gain, k_gain, norm, eps, tok_pos, tok_seq,         \
        page_table, table_width, (T*)k_pages, heads, kv_heads, dim, page_size);                                          \
    values_to_pages_kernel<T, T><<<dim3((max_new + QT_TOKENS - 2) / QT_TOKENS + 1, seqs, kv_heads), 256,                   \
                                   QT_TOKENS * (vdim + 1) * sizeof(float), s>>>(                                          \
        (const T*)proj, (size_t)row_len, (size_t)v_off, cu_seqlens, tok_pos, page_table, table_width, (T*)v_pages,        \
        kv_heads, vdim, page_size)
        if (act_dtype == RI_F32) { RI_VEC(float); } else { RI_VEC(bf16_t); }
#undef RI_VEC
        RI_LAUNCH_CHECK("qk_pairs_norm_kv_write");
        return 0;
    }
    // (a wavefront takes four heads of a token where the launch still has 64 wavefronts a compute unit then: below
    // that fewer, longer wavefronts do not pay)
    const int all_heads = heads + (paged_values ? 1 : 2) * kv_heads;
    const bool four = (long)tokens * all_heads >= 256L * ri_compute_units();
    const long items = (long)tokens * ((all_heads + (four ? 3 : 0)) / (four ? 4 : 1));
#define RI_PAIRS(T, HPW)                                                                                                \
    qk_pairs_norm_kv_write_kernel<T, T, HPW><<<(unsigned)((items + 3) / 4), 256, 0, s>>>(                                 \
        (T*)proj, (size_t)row_len, q_off, k_off, v_off, inv_freq, rot_dims, q_gain, k_gain, norm, eps, tok_pos, tok_seq,  \
        page_table, table_width, (T*)k_pages, (T*)v_pages, tokens, heads, kv_heads, dim, vdim, page_size, !paged_values)
#define RI_GO(T)                                                                                                        \
    if (four) RI_PAIRS(T, 4); else RI_PAIRS(T, 1);                                                                       \
    if (paged_values) {                                                                                                 \
        dim3 grid((max_new + QT_TOKENS - 2) / QT_TOKENS + 1, seqs, kv_heads);                                            \
        values_to_pages_kernel<T, T><<<grid, 256, QT_TOKENS * (vdim + 1) * sizeof(float), s>>>(                           \
            (const T*)proj, (size_t)row_len, (size_t)v_off, cu_seqlens, tok_pos, page_table, table_width, (T*)v_pages,    \
            kv_heads, vdim, page_size);                                                                                 \
    }
    if (act_dtype == RI_F32) { RI_GO(float) } else { RI_GO(bf16_t) }
#undef RI_GO
#undef RI_PAIRS
    RI_LAUNCH_CHECK("qk_pairs_norm_kv_write");
    return 0;
}
