// Windowed softmax attention whose heads' weights are mixed after the softmax, over the paged cache.
//
//   whole_norm_kv_write:  q and k are RMS-normed over the whole projection (all heads at once, one gain an element);
//                         the normed k goes to the key pages, and k as projected, before the norm, to the value pages
//                         (the values are the keys: there is no value projection); q stays in place, normed;
//   talking_attention:    score_h(i, j) = scale (q_h . k_j) - r1_h ln(1 + r2_h (i - j)) for the keys j with 0 <= i - j <
//                         window; w_h = softmax_j(score_h); then the heads talk: w'_h(j) = sum_g T[h, g] w_g(j); head h
//                         applies w'_h to the values of its own key/value head.
//
// The mixing needs every head's finished softmax, so the keys are walked twice: first each head's maximum and sum, a
// workgroup per (token, head); then a workgroup per token makes, tile by tile, the weights of all heads, their mix and
// the products with the values.  Tiles start at fixed multiples (256 keys in the first walk, 32 in the second), so the
// order of every sum depends on the key's position alone.  A step of few tokens cuts the second walk's tiles into shares
// that run side by side and whose float32 results the caller adds.  Scores, the logarithm, softmax statistics, the mix
// and the accumulators are float32.
#include "api.h"
#include "common.h"

#define TK_TILE 32
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

// ------------------------------------------------------------------ the attention itself, in two launches
// 16 bytes of a key row at once where a row starts on a 16-byte boundary.
template <typename TC> struct TkVec;
template <> struct TkVec<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct TkVec<bf16_t> {
    static constexpr int N = 8;
    __device__ static void load(const bf16_t* p, float* o) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = __uint_as_float(w[i] << 16);
            o[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        }
    }
};

#define TK_STAT_TILE 256
#define TK_SUB 8             // query heads of one key head that a thread scores from one load of the key

// The first walk: a workgroup per (token, head) finds the head's maximum and sum over the window; a thread a key, tiles
// of 256 keys that start at multiples of 256.
template <typename TA, typename TC, bool VEC>
__global__ void __launch_bounds__(TK_STAT_TILE)
talking_stats_kernel(float* __restrict__ stats, const TA* __restrict__ q, int q_stride, int q_off,
                     const TC* __restrict__ k_pages, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                     const int32_t* __restrict__ page_table, int table_width, int heads, int kv_heads, int dim, int page_size,
                     int window, float scale, const float* __restrict__ r1, const float* __restrict__ r2) {
    extern __shared__ float qs[];                 // [dim]
    __shared__ float scratch[16];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int kvh = h / (heads / kv_heads);
    const int qpos = tok_pos[t];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int32_t* table = page_table + (size_t)tok_seq[t] * table_width;
    for (int d = tid; d < dim; d += TK_STAT_TILE) qs[d] = to_f32(q[(size_t)t * q_stride + q_off + (size_t)h * dim + d]);
    __syncthreads();
    const float b1 = r1 ? r1[h] : 0.f, b2 = r1 ? r2[h] : 0.f;
    float m = -INFINITY, l = 0.f;
    for (int tile = lo / TK_STAT_TILE; tile <= qpos / TK_STAT_TILE; ++tile) {
        const int j = tile * TK_STAT_TILE + tid;
        const bool valid = j >= lo && j <= qpos;
        float s = -INFINITY;
        if (valid) {
            const TC* kr = k_pages + (((long)table[j / page_size] * kv_heads + kvh) * page_size + j % page_size) * (long)dim;
            float dot = 0.f;
            if (VEC) {
                for (int d = 0; d < dim; d += TkVec<TC>::N) {
                    float kv[TkVec<TC>::N];
                    TkVec<TC>::load(kr + d, kv);
#pragma unroll
                    for (int e = 0; e < TkVec<TC>::N; ++e) dot += qs[d + e] * kv[e];
                }
            } else {
                for (int d = 0; d < dim; ++d) dot += qs[d] * to_f32(kr[d]);
            }
            s = dot * scale;
            if (r1) s -= b1 * log1pf(b2 * (float)(qpos - j));
        }
        const float m_new = fmaxf(m, block_max(s, scratch));          // every tile of the walk holds a visible key
        l = l * expf(m - m_new) + block_sum(valid ? expf(s - m_new) : 0.f, scratch);      // the factor is 0 at the first tile
        m = m_new;
    }
    if (tid == 0) {
        stats[((size_t)t * heads + h) * 2] = m;
        stats[((size_t)t * heads + h) * 2 + 1] = l;
    }
}

// The second walk: a workgroup per token (and share of the key tiles) makes the weights of all heads for a tile of 32
// keys from the first walk's maxima and sums, mixes them, and adds the products with the values.  With more than one
// share the results are partial sums (float32, [share][token][heads * dim]) that the caller adds.
template <typename TA, typename TC, typename TO, bool VEC>
__global__ void __launch_bounds__(256)
talking_mix_kernel(TO* __restrict__ out, int out_stride, int out_off, float out_scale, size_t share_stride,
                   const float* __restrict__ stats, const TA* __restrict__ q, int q_stride, int q_off,
                   const TC* __restrict__ k_pages, const TC* __restrict__ v_pages, const int32_t* __restrict__ tok_pos,
                   const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width, int heads,
                   int kv_heads, int dim, int page_size, int window, float scale, const float* __restrict__ r1,
                   const float* __restrict__ r2, const float* __restrict__ talk) {
    extern __shared__ float lds[];
    float* qs = lds;                                  // [heads * dim]
    float* ps = qs + (size_t)heads * dim;             // [heads][TK_TILE] weights
    float* mixed = ps + (size_t)heads * TK_TILE;      // [heads][TK_TILE]
    float* ms = mixed + (size_t)heads * TK_TILE;      // [heads] maxima
    float* ls = ms + heads;                           // [heads] 1 / sums
    float* tk = ls + heads;                           // [heads][heads] the mixing matrix
    const int t = blockIdx.x, tid = threadIdx.x;
    const int qpos = tok_pos[t];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int share = heads / kv_heads;
    const int sub = share < TK_SUB ? share : TK_SUB;          // heads a thread scores together
    const int subs_per_kv = (share + sub - 1) / sub;
    const int32_t* table = page_table + (size_t)tok_seq[t] * table_width;
    for (int e = tid; e < heads * dim; e += 256) qs[e] = to_f32(q[(size_t)t * q_stride + q_off + e]);
    for (int g = tid; g < heads; g += 256) {
        ms[g] = stats[((size_t)t * heads + g) * 2];
        ls[g] = 1.0f / stats[((size_t)t * heads + g) * 2 + 1];
    }
    if (talk) for (int e = tid; e < heads * heads; e += 256) tk[e] = talk[e];
    __syncthreads();

    const int vdim = dim, results = heads * vdim;
    float acc[TK_ACCS];
#pragma unroll
    for (int i = 0; i < TK_ACCS; ++i) acc[i] = 0.f;
    const int first_tile = lo / TK_TILE, last_tile = qpos / TK_TILE;
    for (int tile = first_tile + blockIdx.y; tile <= last_tile; tile += gridDim.y) {
        const int base = tile * TK_TILE;
        // the weights: a thread takes a key and up to TK_SUB heads of one key head
        for (int item = tid; item < kv_heads * subs_per_kv * TK_TILE; item += 256) {
            const int jj = item % TK_TILE, sg = item / TK_TILE;
            const int kvh = sg / subs_per_kv, g0 = kvh * share + (sg % subs_per_kv) * sub;
            const int n = min(sub, kvh * share + share - g0);
            const int j = base + jj;
            const bool valid = j >= lo && j <= qpos;
            float dots[TK_SUB];
#pragma unroll
            for (int i = 0; i < TK_SUB; ++i) dots[i] = 0.f;
            if (valid) {
                const TC* kr = k_pages + (((long)table[j / page_size] * kv_heads + kvh) * page_size + j % page_size) * (long)dim;
                if (VEC) {
                    // (the heads behind n are the group's last head again: no branch inside the walk over the key, whose
                    // loads go out two at a time)
                    constexpr int N = TkVec<TC>::N;
                    int d = 0;
                    for (; d + 2 * N <= dim; d += 2 * N) {
                        float ka[N], kb[N];
                        TkVec<TC>::load(kr + d, ka);
                        TkVec<TC>::load(kr + d + N, kb);
#pragma unroll
                        for (int i = 0; i < TK_SUB; ++i) {
                            const float* qh = qs + (size_t)(g0 + min(i, n - 1)) * dim + d;
#pragma unroll
                            for (int e = 0; e < N; ++e) dots[i] += qh[e] * ka[e];
#pragma unroll
                            for (int e = 0; e < N; ++e) dots[i] += qh[N + e] * kb[e];
                        }
                    }
                    for (; d < dim; d += N) {
                        float ka[N];
                        TkVec<TC>::load(kr + d, ka);
#pragma unroll
                        for (int i = 0; i < TK_SUB; ++i) {
                            const float* qh = qs + (size_t)(g0 + min(i, n - 1)) * dim + d;
#pragma unroll
                            for (int e = 0; e < N; ++e) dots[i] += qh[e] * ka[e];
                        }
                    }
                } else {
                    for (int d = 0; d < dim; ++d) {
                        const float kv = to_f32(kr[d]);
#pragma unroll
                        for (int i = 0; i < TK_SUB; ++i)
                            if (i < n) dots[i] += qs[(size_t)(g0 + i) * dim + d] * kv;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < TK_SUB; ++i) {
                if (i < n) {
                    const int g = g0 + i;
                    float p = 0.f;
                    if (valid) {
                        float s = dots[i] * scale;
                        if (r1) s -= r1[g] * log1pf(r2[g] * (float)(qpos - j));
                        p = expf(s - ms[g]) * ls[g];
                    }
                    ps[g * TK_TILE + jj] = p;
                }
            }
        }
        __syncthreads();
        // the mix
        for (int item = tid; item < heads * TK_TILE; item += 256) {
            const int jj = item % TK_TILE, h = item / TK_TILE;
            float v;
            if (talk) {
                v = 0.f;
                for (int g = 0; g < heads; ++g) v += tk[h * heads + g] * ps[g * TK_TILE + jj];
            } else {
                v = ps[item];
            }
            mixed[item] = v;
        }
        __syncthreads();
        // the values: eight neighbouring keys of a channel lie side by side in a page
        const int jj_lo = max(lo, base) - base, jj_hi = min(qpos, base + TK_TILE - 1) - base;
        if (page_size % 8 == 0) {
            // eight keys at a time: their page looked up once, then the loads of all of a thread's results asked for
            // before the first is used (a result behind the last is the last again, and dropped)
            for (int j0 = jj_lo & ~7; j0 <= jj_hi; j0 += 8) {
                const int jk = base + j0;
                const long page_at = (long)table[jk / page_size] * kv_heads;
                const int slot = jk % page_size;
#pragma unroll
                for (int i0 = 0; i0 < TK_ACCS; i0 += 4) {
                    if (tid + i0 * 256 >= results) break;          // (the same for the whole workgroup but its last threads)
                    float vv[4][8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int oc = min(tid + (i0 + i) * 256, results - 1);
                        const int h = oc / vdim, c = oc % vdim;
                        const TC* vp = v_pages + ((page_at + h / share) * (long)vdim + c) * page_size + slot;
                        TkVec<TC>::load(vp, vv[i]);
                        if (TkVec<TC>::N == 4) TkVec<TC>::load(vp + 4, vv[i] + 4);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int oc = min(tid + (i0 + i) * 256, results - 1);
                        const float* mx = mixed + (oc / vdim) * TK_TILE + j0;
                        float a = acc[i0 + i];
#pragma unroll
                        for (int e = 0; e < 8; ++e) a += mx[e] * vv[i][e];       // a key that is not seen has the weight 0
                        acc[i0 + i] = a;
                    }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < TK_ACCS; ++i) {
                const int oc = tid + i * 256;
                if (oc < results) {
                    const int h = oc / vdim, c = oc % vdim;
                    float a = acc[i];
                    for (int jj = jj_lo; jj <= jj_hi; ++jj) {
                        const int jk = base + jj;
                        a += mixed[h * TK_TILE + jj] *
                             to_f32(v_pages[(((long)table[jk / page_size] * kv_heads + h / share) * (long)vdim + c) * page_size +
                                            jk % page_size]);
                    }
                    acc[i] = a;
                }
            }
        }
        __syncthreads();                                   // before the next tile overwrites ps and mixed
    }
#pragma unroll
    for (int i = 0; i < TK_ACCS; ++i) {
        const int oc = tid + i * 256;
        if (oc < results)
            from_f32(out + blockIdx.y * share_stride + (size_t)t * out_stride + out_off + oc, acc[i] * out_scale);
    }
}

// How many shares of the key tiles a step's second walk is cut into: one where the tokens alone fill the machine.
extern "C" int ri_talking_attention_shares(int tokens, int longest) {
    if (tokens >= 128) return 1;
    int shares = (longest + TK_TILE - 1) / TK_TILE;
    const int most = (512 + tokens - 1) / tokens;
    if (shares > most) shares = most;
    if (shares > 64) shares = 64;
    return shares < 1 ? 1 : shares;
}

extern "C" int ri_talking_attention(void* out, int out_dtype, int out_stride, int out_off, float out_scale, int shares,
                                    float* stats, const void* q, int act_dtype, int q_stride, int q_off, const void* k_pages,
                                    const void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                                    const int32_t* page_table, int table_width, int tokens, int heads, int kv_heads, int dim,
                                    int page_size, int window, float scale, const float* r1, const float* r2,
                                    const float* talk, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0,
               "talking_attention: %d tokens, %d heads, %d kv heads of %d", tokens, heads, kv_heads, dim);
    RI_REQUIRE((long)heads * dim <= 256L * TK_ACCS, "talking_attention: %d heads of %d exceed the kernel's %d results a token", heads,
               dim, 256 * TK_ACCS);
    RI_REQUIRE(q_off >= 0 && q_off + heads * dim <= q_stride && out_off >= 0 && out_off + heads * dim <= out_stride,
               "talking_attention: columns %d of %d and %d of %d", q_off, q_stride, out_off, out_stride);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16), "talking_attention: dtypes %d and %d",
               act_dtype, cache_dtype);
    RI_REQUIRE(shares >= 1 && shares <= 65535 && (shares == 1 ? out_dtype == act_dtype : out_dtype == RI_F32) && stats,
               "talking_attention: %d shares of the keys with results of dtype %d", shares, out_dtype);
    RI_REQUIRE((r1 == nullptr) == (r2 == nullptr), "talking_attention: the distance bias has two numbers a head");
    RI_REQUIRE(page_size > 0 && table_width > 0 && window >= 0, "talking_attention: page geometry");
    const size_t lds = ((size_t)heads * dim + 2 * (size_t)heads * TK_TILE + 2 * (size_t)heads + (size_t)heads * heads) * sizeof(float);
    RI_REQUIRE(lds <= 64 * 1024, "talking_attention: %d heads of %d need %zu bytes of LDS", heads, dim, lds);
    hipStream_t s = (hipStream_t)stream;
    const bool vec = dim % (act_dtype == RI_F32 ? 4 : 8) == 0 && (uintptr_t)k_pages % 16 == 0 && (uintptr_t)v_pages % 16 == 0;
    const size_t share_stride = (size_t)tokens * out_stride;
#define RI_GO(T, TO, V)                                                                                                     \
    do {                                                                                                                    \
        talking_stats_kernel<T, T, V><<<dim3(tokens, heads), TK_STAT_TILE, (size_t)dim * sizeof(float), s>>>(                \
            stats, (const T*)q, q_stride, q_off, (const T*)k_pages, tok_pos, tok_seq, page_table, table_width, heads, kv_heads, \
            dim, page_size, window, scale, r1, r2);                                                                         \
        talking_mix_kernel<T, T, TO, V><<<dim3(tokens, shares), 256, lds, s>>>(                                              \
            (TO*)out, out_stride, out_off, out_scale, share_stride, stats, (const T*)q, q_stride, q_off, (const T*)k_pages,  \
            (const T*)v_pages, tok_pos, tok_seq, page_table, table_width, heads, kv_heads, dim, page_size, window, scale, r1, \
            r2, talk);                                                                                                      \
    } while (0)
    if (act_dtype == RI_F32) { if (vec) RI_GO(float, float, true); else RI_GO(float, float, false); }
    else if (out_dtype == RI_F32) { if (vec) RI_GO(bf16_t, float, true); else RI_GO(bf16_t, float, false); }
    else { if (vec) RI_GO(bf16_t, bf16_t, true); else RI_GO(bf16_t, bf16_t, false); }
#undef RI_GO
    RI_LAUNCH_CHECK("talking_attention");
    return 0;
}
