// Windowed softmax attention whose heads' weights are mixed after the softmax, over the paged cache.
//
//   whole_norm_kv_write:  q and k are RMS-normed over the whole projection (all heads at once, one gain an element);
//                         the normed k goes to the key pages, and k as projected, before the norm, to the value pages
//                         (the values are the keys: there is no value projection); q stays in place, normed;
//   talking_attention:    score_h(i, j) = scale (q_h . k_j) - r1_h ln(1 + r2_h (i - j)) for the keys j with 0 <= i - j <
//                         window; w_h = softmax_j(score_h); then the heads talk: w'_h(j) = sum_g T[h, g] w_g(j); head h
//                         applies w'_h to the values of its own key/value head.
//
// The mixing needs every head's finished softmax, so a token's heads are one workgroup and the keys are walked twice:
// first each head's maximum and sum (tiles of 64 keys that start at multiples of 64, so the order of every sum depends
// on the key's position alone), then, tile by tile, the weights of all heads, their mix, and the products with the
// values.  Scores, the logarithm, softmax statistics, the mix and the accumulators are float32.
#include "api.h"
#include "common.h"

#define TK_TILE 64
#define TK_ACCS 16           // results a thread accumulates: heads * vdim <= 256 * TK_ACCS

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
whole_norm_kv_write_kernel(TA* __restrict__ proj, int stride, int q_off, int k_off, const float* __restrict__ q_gain,
                           const float* __restrict__ k_gain, float eps, const int32_t* __restrict__ tok_pos,
                           const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width,
                           TC* __restrict__ k_pages, TC* __restrict__ v_pages, int page_size, int heads, int kv_heads, int dim) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int pos = tok_pos[t];
    TA* row = proj + (size_t)t * stride;
    const long page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    const int slot = pos % page_size;
    const int qw = heads * dim, kw = kv_heads * dim;
    float ss = 0.f;
    for (int e = tid; e < qw; e += 256) {
        const float v = to_f32(row[q_off + e]);
        ss += v * v;
    }
    const float q_inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)qw + eps);
    ss = 0.f;
    for (int e = tid; e < kw; e += 256) {
        const float v = to_f32(row[k_off + e]);
        ss += v * v;
    }
    const float k_inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kw + eps);
    for (int e = tid; e < qw; e += 256) from_f32(row + q_off + e, to_f32(row[q_off + e]) * q_inv * q_gain[e]);
    for (int e = tid; e < kw; e += 256) {
        const int g = e / dim, c = e % dim;
        const float v = to_f32(row[k_off + e]);
        from_f32(k_pages + ((page * kv_heads + g) * page_size + slot) * (long)dim + c, v * k_inv * k_gain[e]);
        from_f32(v_pages + ((page * kv_heads + g) * (long)dim + c) * page_size + slot, v);
    }
}

extern "C" int ri_whole_norm_kv_write(void* proj, int act_dtype, int stride, int q_off, int k_off, const float* q_gain,
                                      const float* k_gain, float eps, const int32_t* tok_pos, const int32_t* tok_seq,
                                      const int32_t* page_table, int table_width, void* k_pages, void* v_pages, int cache_dtype,
                                      int page_size, int tokens, int heads, int kv_heads, int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && dim > 0, "whole_norm_kv_write: %d tokens, %d and %d heads of %d", tokens,
               heads, kv_heads, dim);
    RI_REQUIRE(q_off >= 0 && k_off >= 0 && q_off + heads * dim <= stride && k_off + kv_heads * dim <= stride,
               "whole_norm_kv_write: columns %d and %d of rows of %d", q_off, k_off, stride);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16), "whole_norm_kv_write: dtypes %d and %d",
               act_dtype, cache_dtype);
    RI_REQUIRE(page_size > 0 && table_width > 0 && q_gain && k_gain, "whole_norm_kv_write: page geometry and gains");
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        whole_norm_kv_write_kernel<float, float><<<tokens, 256, 0, s>>>((float*)proj, stride, q_off, k_off, q_gain, k_gain, eps,
                                                                       tok_pos, tok_seq, page_table, table_width, (float*)k_pages,
                                                                       (float*)v_pages, page_size, heads, kv_heads, dim);
    else
        whole_norm_kv_write_kernel<bf16_t, bf16_t><<<tokens, 256, 0, s>>>((bf16_t*)proj, stride, q_off, k_off, q_gain, k_gain, eps,
                                                                         tok_pos, tok_seq, page_table, table_width,
                                                                         (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, heads,
                                                                         kv_heads, dim);
    RI_LAUNCH_CHECK("whole_norm_kv_write");
    return 0;
}

// The raw score of head g for the key at position j (which the caller has found visible).
template <typename TC>
__device__ __forceinline__ float talking_score(const float* __restrict__ qs, const TC* __restrict__ k_pages,
                                               const int32_t* __restrict__ table, int g, int j, int qpos, int share,
                                               int kv_heads, int dim, int page_size, float scale, const float* r1,
                                               const float* r2) {
    const long page = table[j / page_size];
    const TC* kr = k_pages + ((page * kv_heads + g / share) * page_size + j % page_size) * (long)dim;
    const float* qh = qs + (size_t)g * dim;
    float dot = 0.f;
    for (int d = 0; d < dim; ++d) dot += qh[d] * to_f32(kr[d]);
    float s = dot * scale;
    if (r1) s -= r1[g] * log1pf(r2[g] * (float)(qpos - j));
    return s;
}

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
talking_attention_kernel(TA* __restrict__ out, int out_stride, int out_off, float out_scale, const TA* __restrict__ q,
                         int q_stride, int q_off, const TC* __restrict__ k_pages, const TC* __restrict__ v_pages,
                         const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                         const int32_t* __restrict__ page_table, int table_width, int heads, int kv_heads, int dim,
                         int page_size, int window, float scale, const float* __restrict__ r1, const float* __restrict__ r2,
                         const float* __restrict__ talk) {
    extern __shared__ float lds[];
    float* qs = lds;                                  // [heads * dim]
    float* ps = qs + (size_t)heads * dim;             // [heads][TK_TILE]: scores, then weights
    float* mixed = ps + (size_t)heads * TK_TILE;      // [heads][TK_TILE]
    float* ms = mixed + (size_t)heads * TK_TILE;      // [heads] maxima
    float* ls = ms + heads;                           // [heads] sums
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qpos = tok_pos[t];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int share = heads / kv_heads;
    const int32_t* table = page_table + (size_t)tok_seq[t] * table_width;
    for (int e = tid; e < heads * dim; e += 256) qs[e] = to_f32(q[(size_t)t * q_stride + q_off + e]);
    __syncthreads();

    const int first_tile = lo / TK_TILE, last_tile = qpos / TK_TILE;
    // the first walk: every head's maximum and sum; a wavefront takes a head and its 64 scores of every tile
    for (int g = wave; g < heads; g += 4) {
        float m = -INFINITY, l = 0.f;
        for (int tile = first_tile; tile <= last_tile; ++tile) {
            const int j = tile * TK_TILE + lane;
            const bool valid = j >= lo && j <= qpos;
            const float s = valid ? talking_score(qs, k_pages, table, g, j, qpos, share, kv_heads, dim, page_size, scale, r1, r2)
                                  : -INFINITY;
            const float m_new = fmaxf(m, wave_max(s));             // every tile of the walk holds a visible key
            l = l * expf(m - m_new) + wave_sum(valid ? expf(s - m_new) : 0.f);      // the factor is 0 at the first tile
            m = m_new;
        }
        if (lane == 0) { ms[g] = m; ls[g] = l; }
    }
    __syncthreads();

    // the second walk: the weights of all heads for a tile, their mix, the products with the values
    const int vdim = dim, results = heads * vdim;
    float acc[TK_ACCS];
#pragma unroll
    for (int i = 0; i < TK_ACCS; ++i) acc[i] = 0.f;
    for (int tile = first_tile; tile <= last_tile; ++tile) {
        const int base = tile * TK_TILE;
        const int j = base + lane;
        const bool valid = j >= lo && j <= qpos;
        for (int g = wave; g < heads; g += 4) {
            float p = 0.f;
            if (valid) {
                const float s = talking_score(qs, k_pages, table, g, j, qpos, share, kv_heads, dim, page_size, scale, r1, r2);
                p = expf(s - ms[g]) / ls[g];
            }
            ps[g * TK_TILE + lane] = p;
        }
        __syncthreads();
        for (int h = wave; h < heads; h += 4) {
            float v = 0.f;
            if (talk) {
                for (int g = 0; g < heads; ++g) v += talk[h * heads + g] * ps[g * TK_TILE + lane];
            } else {
                v = ps[h * TK_TILE + lane];
            }
            mixed[h * TK_TILE + lane] = v;
        }
        __syncthreads();
        const int jj_lo = max(lo, base) - base, jj_hi = min(qpos, base + TK_TILE - 1) - base;
#pragma unroll
        for (int i = 0; i < TK_ACCS; ++i) {
            const int oc = tid + i * 256;
            if (oc < results) {
                const int h = oc / vdim, c = oc % vdim;
                float a = acc[i];
                for (int jj = jj_lo; jj <= jj_hi; ++jj) {
                    const int jk = base + jj;
                    const long page = table[jk / page_size];
                    a += mixed[h * TK_TILE + jj] *
                         to_f32(v_pages[((page * kv_heads + h / share) * (long)vdim + c) * page_size + jk % page_size]);
                }
                acc[i] = a;
            }
        }
        __syncthreads();                                   // before the next tile overwrites ps and mixed
    }
#pragma unroll
    for (int i = 0; i < TK_ACCS; ++i) {
        const int oc = tid + i * 256;
        if (oc < results) from_f32(out + (size_t)t * out_stride + out_off + oc, acc[i] * out_scale);
    }
}

extern "C" int ri_talking_attention(void* out, int out_stride, int out_off, float out_scale, const void* q, int act_dtype,
                                    int q_stride, int q_off, const void* k_pages, const void* v_pages, int cache_dtype,
                                    const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table, int table_width,
                                    int tokens, int heads, int kv_heads, int dim, int page_size, int window, float scale,
                                    const float* r1, const float* r2, const float* talk, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0,
               "talking_attention: %d tokens, %d heads, %d kv heads of %d", tokens, heads, kv_heads, dim);
    RI_REQUIRE((long)heads * dim <= 256L * TK_ACCS, "talking_attention: %d heads of %d exceed the kernel's %d results a token", heads,
               dim, 256 * TK_ACCS);
    RI_REQUIRE(q_off >= 0 && q_off + heads * dim <= q_stride && out_off >= 0 && out_off + heads * dim <= out_stride,
               "talking_attention: columns %d of %d and %d of %d", q_off, q_stride, out_off, out_stride);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16), "talking_attention: dtypes %d and %d",
               act_dtype, cache_dtype);
    RI_REQUIRE((r1 == nullptr) == (r2 == nullptr), "talking_attention: the distance bias has two numbers a head");
    RI_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "talking_attention: page geometry");
    const size_t lds = ((size_t)heads * dim + 2 * (size_t)heads * TK_TILE + 2 * (size_t)heads) * sizeof(float);
    RI_REQUIRE(lds <= 64 * 1024, "talking_attention: %d heads of %d need %zu bytes of LDS", heads, dim, lds);
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        talking_attention_kernel<float, float><<<tokens, 256, lds, s>>>(
            (float*)out, out_stride, out_off, out_scale, (const float*)q, q_stride, q_off, (const float*)k_pages,
            (const float*)v_pages, tok_pos, tok_seq, page_table, table_width, heads, kv_heads, dim, page_size, window, scale, r1,
            r2, talk);
    else
        talking_attention_kernel<bf16_t, bf16_t><<<tokens, 256, lds, s>>>(
            (bf16_t*)out, out_stride, out_off, out_scale, (const bf16_t*)q, q_stride, q_off, (const bf16_t*)k_pages,
            (const bf16_t*)v_pages, tok_pos, tok_seq, page_table, table_width, heads, kv_heads, dim, page_size, window, scale, r1,
            r2, talk);
    RI_LAUNCH_CHECK("talking_attention");
    return 0;
}
