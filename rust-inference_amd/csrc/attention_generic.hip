// Causal grouped-query attention over the paged cache for any number of new tokens per sequence:
// the form every other attention kernel here is checked against, and the one the float32 path runs.
// One workgroup per (token, query head); keys in tiles of 256 that start at multiples of 256, so the
// order of every sum depends on the key's position alone, never on how tokens were cut into steps.
//
// score_j = (q . k_j) * scale, then, with a cap c > 0, score_j <- c tanh(score_j / c), then, with a slope per
// query head, score_j <- score_j - slope_h (p - j); the query at position p
// sees keys lo..p with lo = 0 or p - window + 1, and with keep_first > 0 also the keys 0..keep_first-1 that lie
// before lo (the first tokens of a sequence stay visible behind the window); with a sink per query head the
// softmax's denominator also holds exp(sink_h), which has no key and no value;
// online softmax with running maximum m, running sum l and factor exp(m_old - m_new)
// (the reference: src/attention.rs:117-149; its GPU form src/cuda/kernels.cu:345-405).
//
// Any head size from 1 to 1,024 (the reference asks only that it be even, and only because of its rotation:
// src/models/config.rs:98-100; its own attention test runs head size 8, src/attention.rs:189-219): keys are
// read 16 bytes at a time where a key row starts on a 16-byte boundary (head sizes that are multiples of 4
// in float32, of 8 in bfloat16) and element by element otherwise; a thread accumulates up to four channels.
// The value heads may have another size (v_dim) than the query and key heads.
#include "api.h"
#include "common.h"

#define ATT_TILE 256

template <typename TC> struct Vec;
template <> struct Vec<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct Vec<bf16_t> {
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

#define ATT_ACCS 4                              // channels of a value head a thread accumulates
#define ATT_MAX_HEAD_DIM (ATT_ACCS * ATT_TILE)

template <typename TA, typename TC, bool VEC>
__global__ void __launch_bounds__(ATT_TILE)
attention_generic_kernel(TA* __restrict__ out, const TA* __restrict__ q, int q_stride, const TC* __restrict__ k_pages,
                         const TC* __restrict__ v_pages, const int32_t* __restrict__ tok_pos,
                         const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ page_table, int table_width,
                         int heads, int kv_heads, int head_dim, int v_dim, int page_size, int window, float scale,
                         float softcap, const float* __restrict__ slopes, int keep_first,
                         const float* __restrict__ sinks) {
    extern __shared__ float qs[];                 // head_dim floats: the query
    __shared__ float ps[ATT_TILE];                // this tile's weights
    __shared__ long rowoff[ATT_TILE];             // element offset of each key's column in the value pool
    __shared__ float scratch[16];

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int kvh = h / (heads / kv_heads);       // consecutive query heads share a kv head
    const int qpos = tok_pos[t];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const float slope = slopes ? slopes[h] : 0.f;
    const int32_t* table = page_table + (size_t)tok_seq[t] * table_width;

    for (int d = tid; d < head_dim; d += ATT_TILE) qs[d] = to_f32(q[(size_t)t * q_stride + (size_t)h * head_dim + d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f, acc = 0.f, acc2 = 0.f;      // channels tid and tid + 256
    float acc3 = 0.f, acc4 = 0.f;                              // and tid + 512, tid + 768 (value heads above 512)
    const int kept = min(keep_first, lo);         // keys 0..kept-1 are seen although they lie behind the window
    const int lo_tile = lo / ATT_TILE, kept_tiles = (kept + ATT_TILE - 1) / ATT_TILE;
    for (int tile = 0; tile <= qpos / ATT_TILE; ++tile) {
        if (tile >= kept_tiles && tile < lo_tile) { tile = lo_tile - 1; continue; }      // (the same for the whole workgroup)
        const int j = tile * ATT_TILE + tid;
        const bool valid = (j >= lo || j < kept) && j <= qpos;
        float s = -INFINITY;
        if (valid) {
            const long page_head = ((long)table[j / page_size] * kv_heads + kvh) * page_size;
            const long head_base = page_head * head_dim;
            rowoff[tid] = page_head * v_dim + j % page_size;       // the key's column in the transposed value page
            const TC* kr = k_pages + head_base + (long)(j % page_size) * head_dim;
            float dot = 0.f;
            if (VEC) {
                for (int d = 0; d < head_dim; d += Vec<TC>::N) {
                    float kv[Vec<TC>::N];
                    Vec<TC>::load(kr + d, kv);
#pragma unroll
                    for (int e = 0; e < Vec<TC>::N; ++e) dot += qs[d + e] * kv[e];
                }
            } else {
                for (int d = 0; d < head_dim; ++d) dot += qs[d] * to_f32(kr[d]);      // the same order of additions
            }
            s = dot * scale;
            if (softcap > 0.f) s = softcap * tanhf(s / softcap);
            if (slopes) s -= slope * (float)(qpos - j);
        }
        const float m_new = fmaxf(m, block_max(s, scratch));
        const float p = valid ? expf(s - m_new) : 0.f;
        ps[tid] = p;
        const float tile_sum = block_sum(p, scratch);      // its barriers also publish ps and rowoff
        const float corr = expf(m - m_new);                // 0 on the first tile (m = -inf)
        l = l * corr + tile_sum;
        m = m_new;
        if (tid < v_dim) {
            acc *= corr;
            acc2 *= corr;
            acc3 *= corr;
            acc4 *= corr;
            const int base = tile * ATT_TILE;
            const int last = min(qpos, base + ATT_TILE - 1) - base;
            const bool second = tid + ATT_TILE < v_dim, third = tid + 2 * ATT_TILE < v_dim, fourth = tid + 3 * ATT_TILE < v_dim;
            if (VEC && page_size % 8 == 0) {
                // eight neighbouring keys of a channel lie side by side in a value page: one 16-byte load (two in
                // float32) instead of eight elements; a key that is not seen has the weight 0
                for (int j0 = 0; j0 <= last; j0 += 8) {
                    const int a = base + j0, b = min(a + 7, qpos);
                    if (b < lo && a >= kept) continue;                         // none of the eight is seen
                    const TC* vp = v_pages + ((long)table[a / page_size] * kv_heads + kvh) * page_size * (long)v_dim +
                                   a % page_size + (long)tid * page_size;
                    float vv[8];
                    Vec<TC>::load(vp, vv);
                    if (Vec<TC>::N == 4) Vec<TC>::load(vp + 4, vv + 4);
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc += ps[j0 + e] * vv[e];
                    if (second) {
                        Vec<TC>::load(vp + (long)ATT_TILE * page_size, vv);
                        if (Vec<TC>::N == 4) Vec<TC>::load(vp + (long)ATT_TILE * page_size + 4, vv + 4);
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc2 += ps[j0 + e] * vv[e];
                    }
                    if (third) {
                        Vec<TC>::load(vp + 2L * ATT_TILE * page_size, vv);
                        if (Vec<TC>::N == 4) Vec<TC>::load(vp + 2L * ATT_TILE * page_size + 4, vv + 4);
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc3 += ps[j0 + e] * vv[e];
                    }
                    if (fourth) {
                        Vec<TC>::load(vp + 3L * ATT_TILE * page_size, vv);
                        if (Vec<TC>::N == 4) Vec<TC>::load(vp + 3L * ATT_TILE * page_size + 4, vv + 4);
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc4 += ps[j0 + e] * vv[e];
                    }
                }
            } else
            for (int jj = 0; jj <= last; ++jj) {
                if (base + jj < lo && base + jj >= kept) continue;         // not seen: no weight, and no offset either
                acc += ps[jj] * to_f32(v_pages[rowoff[jj] + (long)tid * page_size]);
                if (second) acc2 += ps[jj] * to_f32(v_pages[rowoff[jj] + (long)(tid + ATT_TILE) * page_size]);
                if (third) acc3 += ps[jj] * to_f32(v_pages[rowoff[jj] + (long)(tid + 2 * ATT_TILE) * page_size]);
                if (fourth) acc4 += ps[jj] * to_f32(v_pages[rowoff[jj] + (long)(tid + 3 * ATT_TILE) * page_size]);
            }
        }
        __syncthreads();                                   // before the next tile overwrites ps and rowoff
    }
    if (sinks) l += expf(sinks[h] - m);                    // the sink: a term of the denominator alone
    if (tid < v_dim) from_f32(out + ((size_t)t * heads + h) * v_dim + tid, acc / l);
    if (tid + ATT_TILE < v_dim) from_f32(out + ((size_t)t * heads + h) * v_dim + tid + ATT_TILE, acc2 / l);
    if (tid + 2 * ATT_TILE < v_dim) from_f32(out + ((size_t)t * heads + h) * v_dim + tid + 2 * ATT_TILE, acc3 / l);
    if (tid + 3 * ATT_TILE < v_dim) from_f32(out + ((size_t)t * heads + h) * v_dim + tid + 3 * ATT_TILE, acc4 / l);
}

template <typename T, bool VEC>
static void launch_attention(void* out, const void* q, int q_stride, const void* k_pages, const void* v_pages,
                             const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                             int table_width, int tokens, int heads, int kv_heads, int head_dim, int v_dim,
                             int page_size, int window, float scale, float softcap, const float* slopes, int keep_first,
                             const float* sinks, hipStream_t s) {
    attention_generic_kernel<T, T, VEC><<<dim3(tokens, heads), ATT_TILE, (size_t)head_dim * sizeof(float), s>>>(
        (T*)out, (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, tok_pos, tok_seq, page_table,
        table_width, heads, kv_heads, head_dim, v_dim, page_size, window, scale, softcap, slopes, keep_first, sinks);
}

extern "C" int ri_attention_kept(void* out, const void* q, int act_dtype, int q_stride, const void* k_pages,
                            const void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                            const int32_t* page_table, int table_width, int tokens, int heads, int kv_heads,
                            int head_dim, int v_dim, int page_size, int window, float scale, float softcap,
                            const float* slopes, int keep_first, const float* sinks, void* stream) {
    RI_REQUIRE(keep_first >= 0, "attention: %d first tokens kept", keep_first);
    RI_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "attention: tokens %d, heads %d, kv heads %d", tokens, heads, kv_heads);
    RI_REQUIRE(head_dim >= 1 && head_dim <= ATT_MAX_HEAD_DIM, "attention: head_dim %d must be between 1 and %d", head_dim,
               ATT_MAX_HEAD_DIM);
    RI_REQUIRE(v_dim >= 1 && v_dim <= ATT_MAX_HEAD_DIM, "attention: value head size %d must be between 1 and %d", v_dim,
               ATT_MAX_HEAD_DIM);
    RI_REQUIRE(heads <= 65535, "attention: %d heads exceed one launch", heads);
    RI_REQUIRE(q_stride >= heads * head_dim, "attention: q row stride %d for %d heads of %d", q_stride, heads, head_dim);
    RI_REQUIRE(act_dtype == cache_dtype && (act_dtype == RI_F32 || act_dtype == RI_BF16),
               "attention: activations (%d) and cache (%d) must share float32 or bfloat16", act_dtype, cache_dtype);
    RI_REQUIRE(page_size > 0 && table_width > 0, "attention: page geometry");
    hipStream_t s = (hipStream_t)stream;
    // a key row starts on a 16-byte boundary when the head size is a multiple of 4 (float32) or 8 (bfloat16):
    // the pools themselves are 256-byte aligned allocations
    const bool vec = head_dim % (act_dtype == RI_F32 ? 4 : 8) == 0 && (uintptr_t)k_pages % 16 == 0 && (uintptr_t)v_pages % 16 == 0;
#define RI_ATT_GO(T, V) launch_attention<T, V>(out, q, q_stride, k_pages, v_pages, tok_pos, tok_seq, page_table, \
                                               table_width, tokens, heads, kv_heads, head_dim, v_dim, page_size, window, scale, \
                                               softcap, slopes, window > 0 ? keep_first : 0, sinks, s)
    if (act_dtype == RI_F32) { if (vec) RI_ATT_GO(float, true); else RI_ATT_GO(float, false); }
    else                     { if (vec) RI_ATT_GO(bf16_t, true); else RI_ATT_GO(bf16_t, false); }
#undef RI_ATT_GO
    RI_LAUNCH_CHECK("attention");
    return 0;
}

extern "C" int ri_attention(void* out, const void* q, int act_dtype, int q_stride, const void* k_pages,
                            const void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                            const int32_t* page_table, int table_width, int tokens, int heads, int kv_heads,
                            int head_dim, int v_dim, int page_size, int window, float scale, float softcap,
                            const float* slopes, void* stream) {
    return ri_attention_kept(out, q, act_dtype, q_stride, k_pages, v_pages, cache_dtype, tok_pos, tok_seq, page_table,
                             table_width, tokens, heads, kv_heads, head_dim, v_dim, page_size, window, scale, softcap,
                             slopes, 0, nullptr, stream);
}
