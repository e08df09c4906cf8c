// Attention over a cached latent: what lies around the attention kernel.
//
// A token's keys and values of all heads are products of one latent vector c (kv_rank numbers) with per-head matrices,
// plus one rotated key part shared by the heads.  Only c and that part are cached, and the attention runs on them
// directly: with k_h = U_h c the score q_h . k_h is (U_h^T q_h) . c, and sum_j w_j (V_h c_j) is V_h (sum_j w_j c_j).  So
// the cache holds, per token, one key row [c | rotated part] and one value row c for a single key/value head, the
// queries become [U_h^T q_h | rotated q_h] (kv_rank + rot numbers a head), and the heads' results (kv_rank numbers) go
// through V_h afterwards.
//
//   latent_prepare:  c = rms_norm(first kv_rank outputs of the down projection) * gain; the last rot outputs and the
//                    last rot elements of every query head turn in neighbouring pairs (2i, 2i + 1) by p * f_i; c and
//                    the turned key part go to the key page, c to the value page (transposed inside a page);
//   head_products:   out[t, h, :] = gate[t, h] * x[t, h, :] W_h for matrices W_h [K, N] of a stack [H, K, N], with the
//                    elements of x behind K copied behind N (the rotated part of a query rides along); the gate is the
//                    sigmoid of one number per token and head, or absent.
//
// Norm statistics, angles, sines and cosines, the gate's sigmoid and every sum are float32.
#include "api.h"
#include "common.h"

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(TA* __restrict__ proj, int stride, int q_off, int kv_off, const float* __restrict__ gain, float eps,
                      const float* __restrict__ inv_freq, const int32_t* __restrict__ tok_pos,
                      const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width,
                      TC* __restrict__ k_pages, TC* __restrict__ v_pages, int page_size, int heads, int dim, int rot, int rank) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int pos = tok_pos[t];
    TA* row = proj + (size_t)t * stride;
    const long page = page_table[(size_t)tok_seq[t] * table_width + pos / page_size];
    const int slot = pos % page_size;
    TC* krow = k_pages + (page * page_size + slot) * (long)(rank + rot);
    TC* vcol = v_pages + page * (long)rank * page_size + slot;
    float ss = 0.f;
    for (int r = tid; r < rank; r += 256) {
        const float v = to_f32(row[kv_off + r]);
        ss += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)rank + eps);
    for (int r = tid; r < rank; r += 256) {
        const float c = to_f32(row[kv_off + r]) * inv * gain[r];
        from_f32(krow + r, c);
        from_f32(vcol + (long)r * page_size, c);
    }
    const int half = rot / 2;
    // the shared key part (one "head") and every query head's last rot elements
    for (int e = tid; e < (heads + 1) * half; e += 256) {
        const int h = e / half, i = e % half;
        const float a = (float)pos * inv_freq[i];
        const float cs = cosf(a), sn = sinf(a);
        if (h == heads) {
            const float u = to_f32(row[kv_off + rank + 2 * i]), v = to_f32(row[kv_off + rank + 2 * i + 1]);
            from_f32(krow + rank + 2 * i, u * cs - v * sn);
            from_f32(krow + rank + 2 * i + 1, v * cs + u * sn);
        } else {
            TA* qp = row + q_off + (size_t)h * (dim + rot) + dim + 2 * i;
            const float u = to_f32(qp[0]), v = to_f32(qp[1]);
            from_f32(qp, u * cs - v * sn);
            from_f32(qp + 1, v * cs + u * sn);
        }
    }
}

extern "C" int ri_latent_prepare(void* proj, int act_dtype, int stride, int q_off, int kv_off, const float* gain, float eps,
                                 const float* inv_freq, const int32_t* tok_pos, const int32_t* tok_seq,
                                 const int32_t* page_table, int table_width, void* k_pages, void* v_pages, int cache_dtype,
                                 int page_size, int tokens, int heads, int dim, int rot, int rank, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && dim >= 0 && rank > 0 && rot >= 0 && rot % 2 == 0,
               "latent_prepare: %d tokens, %d heads of %d + %d, latent %d", tokens, heads, dim, rot, rank);
    RI_REQUIRE(q_off >= 0 && kv_off >= 0 && q_off + heads * (dim + rot) <= stride && kv_off + rank + rot <= stride,
               "latent_prepare: columns %d and %d of rows of %d", q_off, kv_off, stride);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16), "latent_prepare: dtypes %d and %d",
               act_dtype, cache_dtype);
    RI_REQUIRE(rot == 0 || inv_freq, "latent_prepare: a rotation needs its frequencies");
    RI_REQUIRE(page_size > 0 && table_width > 0, "latent_prepare: page geometry");
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == RI_F32)
        latent_prepare_kernel<float, float><<<tokens, 256, 0, s>>>((float*)proj, stride, q_off, kv_off, gain, eps, inv_freq,
                                                                  tok_pos, tok_seq, page_table, table_width, (float*)k_pages,
                                                                  (float*)v_pages, page_size, heads, dim, rot, rank);
    else
        latent_prepare_kernel<bf16_t, bf16_t><<<tokens, 256, 0, s>>>((bf16_t*)proj, stride, q_off, kv_off, gain, eps, inv_freq,
                                                                    tok_pos, tok_seq, page_table, table_width, (bf16_t*)k_pages,
                                                                    (bf16_t*)v_pages, page_size, heads, dim, rot, rank);
    RI_LAUNCH_CHECK("latent_prepare");
    return 0;
}

// ------------------------------------------------------------------ a product per head
#define HP_TOKENS 8          // tokens of a workgroup: a matrix element is loaded once for all of them
#define HP_COLS 64           // result columns of a workgroup
#define HP_SLICES 4          // slices of K that the four wavefronts of a workgroup take: a lane sums its slice's rows in order,
                             // the slices meet through LDS in order

template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(HP_COLS * HP_SLICES)
head_products_kernel(TO* __restrict__ out, int out_stride, int out_off, int out_head, const TX* __restrict__ x, int x_stride,
                     int x_off, int x_head, const TW* __restrict__ w, const TX* __restrict__ gates, int g_stride, int g_off,
                     float scale, int tokens, int k, int n, int extra) {
    extern __shared__ float lds[];
    float* xs = lds;                                          // [HP_TOKENS][k + extra]
    const int width = k + extra;
    float* red = xs + HP_TOKENS * width;                      // [HP_SLICES][HP_TOKENS][HP_COLS]
    const int h = blockIdx.y, t0 = blockIdx.x * HP_TOKENS, tid = threadIdx.x;
    const int lane = tid % HP_COLS, slice = tid / HP_COLS;
    const int c = blockIdx.z * HP_COLS + lane;
    for (int e = tid; e < HP_TOKENS * width; e += HP_COLS * HP_SLICES) {
        const int tt = e / width, col = e % width, t = t0 + tt;
        xs[e] = t < tokens ? to_f32(x[(size_t)t * x_stride + x_off + (size_t)h * x_head + col]) : 0.f;
    }
    __syncthreads();
    float acc[HP_TOKENS];
#pragma unroll
    for (int tt = 0; tt < HP_TOKENS; ++tt) acc[tt] = 0.f;
    if (c < n) {
        const TW* wc = w + (size_t)h * k * n + c;
        const int per = (k + HP_SLICES - 1) / HP_SLICES;      // rows of a slice
        const int r0 = slice * per, r1 = min(k, r0 + per);
        int r = r0;
        for (; r + 8 <= r1; r += 8) {                         // eight loads asked for before the first is used
            float wv[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) wv[i] = to_f32(wc[(size_t)(r + i) * n]);
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int tt = 0; tt < HP_TOKENS; ++tt) acc[tt] += xs[tt * width + r + i] * wv[i];
        }
        for (; r < r1; ++r) {
            const float wv = to_f32(wc[(size_t)r * n]);
#pragma unroll
            for (int tt = 0; tt < HP_TOKENS; ++tt) acc[tt] += xs[tt * width + r] * wv;
        }
    } else if (c < n + extra && slice == 0) {
#pragma unroll
        for (int tt = 0; tt < HP_TOKENS; ++tt) acc[tt] = xs[tt * width + k + (c - n)];
    }
#pragma unroll
    for (int tt = 0; tt < HP_TOKENS; ++tt) red[(slice * HP_TOKENS + tt) * HP_COLS + lane] = acc[tt];
    __syncthreads();
    if (slice == 0 && c < n + extra) {
#pragma unroll
        for (int tt = 0; tt < HP_TOKENS; ++tt) {
            const int t = t0 + tt;
            if (t >= tokens) break;
            float v = red[tt * HP_COLS + lane];
            for (int sl = 1; sl < HP_SLICES; ++sl) v += red[(sl * HP_TOKENS + tt) * HP_COLS + lane];
            float g = scale;
            if (gates) g *= 1.f / (1.f + expf(-to_f32(gates[(size_t)t * g_stride + g_off + h])));
            from_f32(out + (size_t)t * out_stride + out_off + (size_t)h * out_head + c, v * g);
        }
    }
}

extern "C" int ri_head_products(void* out, int out_dtype, int out_stride, int out_off, int out_head, const void* x, int x_dtype,
                                int x_stride, int x_off, int x_head, const void* w, int w_dtype, const void* gates, int g_stride,
                                int g_off, float scale, int tokens, int heads, int k, int n, int extra, void* stream) {
    // k = n = 0: no product, the copied elements alone (with the head's gate and the scale); w is not read
    RI_REQUIRE(tokens > 0 && heads > 0 && heads <= 65535 && extra >= 0 && ((k > 0 && n > 0) || (k == 0 && n == 0 && extra > 0)),
               "head_products: %d tokens, %d heads of %d x %d (+%d)", tokens, heads, k, n, extra);
    RI_REQUIRE(x_off >= 0 && x_head >= k + extra && x_off + (long)(heads - 1) * x_head + k + extra <= x_stride,
               "head_products: heads of %d at column %d of rows of %d", x_head, x_off, x_stride);
    RI_REQUIRE(out_off >= 0 && out_head >= n + extra && out_off + (long)(heads - 1) * out_head + n + extra <= out_stride,
               "head_products: results of %d at column %d of rows of %d", out_head, out_off, out_stride);
    RI_REQUIRE(!gates || (g_off >= 0 && g_off + heads <= g_stride), "head_products: gates at column %d of rows of %d", g_off, g_stride);
    RI_REQUIRE((x_dtype == RI_F32 || x_dtype == RI_BF16) && (w_dtype == RI_F32 || w_dtype == RI_BF16) &&
               (out_dtype == RI_F32 || out_dtype == RI_BF16), "head_products: dtypes %d, %d, %d", x_dtype, w_dtype, out_dtype);
    const size_t lds = ((size_t)HP_TOKENS * (k + extra) + (size_t)HP_SLICES * HP_TOKENS * HP_COLS) * sizeof(float);
    RI_REQUIRE(lds <= 64 * 1024, "head_products: heads of %d exceed the kernel's 1792", k + extra);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((tokens + HP_TOKENS - 1) / HP_TOKENS, heads, (n + extra + HP_COLS - 1) / HP_COLS);
    RI_REQUIRE(grid.z <= 65535, "head_products: results of %d", n + extra);
#define RI_GO(TX, TW, TO)                                                                                               \
    head_products_kernel<TX, TW, TO><<<grid, HP_COLS * HP_SLICES, lds, s>>>((TO*)out, out_stride, out_off, out_head, (const TX*)x, x_stride, \
                                                            x_off, x_head, (const TW*)w, (const TX*)gates, g_stride, g_off, \
                                                            scale, tokens, k, n, extra)
    if (x_dtype == RI_F32) {
        RI_REQUIRE(out_dtype == RI_F32, "head_products: float32 rows give float32 results");
        if (w_dtype == RI_F32) RI_GO(float, float, float); else RI_GO(float, bf16_t, float);
    } else {
        RI_REQUIRE(w_dtype == RI_BF16, "head_products: bfloat16 rows take bfloat16 matrices");
        if (out_dtype == RI_F32) RI_GO(bf16_t, bf16_t, float); else RI_GO(bf16_t, bf16_t, bf16_t);
    }
#undef RI_GO
    RI_LAUNCH_CHECK("head_products");
    return 0;
}
