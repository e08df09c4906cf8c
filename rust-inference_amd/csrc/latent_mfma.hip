// Attention over a cached latent on the matrix cores, for prompts in bfloat16.
//
// The cache entry is one key/value head: key rows [c | rotated part] of DK = 32 KS elements, value rows c of 16 VT
// elements (the first 16 VT of a key row, kept a second time transposed inside a page for the value product).  All query
// heads read it, so a wavefront takes 16 query heads of one token as the 16 columns of its tiles and walks the token's
// pages: scores S^T = K Q^T (KS products a half page), the softmax's running maximum and sum per column, and
// O^T += V^T P^T (VT products a page).  The key rows of a half page are permuted (row r of the first half is key
// 8 (r / 4) + r % 4, of the second that plus 4), so that a lane's eight scores are eight neighbouring keys, which is
// how the value product wants its weights: no exchange between lanes.  A sink per head joins the sum once at the end.
// Scores, maxima, sums and the accumulators are float32; the weights are rounded to bfloat16 for the value product, as
// in this library's other matrix-core attention.  A token's sums run over its pages in order, whatever else the step holds.
// A step of few tokens cuts a token's pages into chunks that wavefronts walk side by side; each leaves its maximum, its sum
// and its sums of values, and a second kernel joins them in the chunks' order.
#include "api.h"
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 lm_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float lm_floatx4;

union LmFrag {
    lm_bf16x8 v;
    uint4 u;
    uint32_t w[4];
};

#define LM_PAGE 32
#define LM_WAVES 4
#define LM_MAX_CHUNKS 64

template <int KS, int VT>
__global__ void __launch_bounds__(64 * LM_WAVES)
latent_attention_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int q_stride,
                             const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                             const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                             const int32_t* __restrict__ page_table, int table_width, int tokens, int heads, int tiles,
                             float scale_log2, const float* __restrict__ sinks, float* __restrict__ partial, int chunks,
                             int chunk_pages) {
    constexpr int DK = 32 * KS, RANK = 16 * VT;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int unit = blockIdx.x * LM_WAVES + wave;            // (token, tile of 16 heads, chunk of pages)
    if (unit >= tokens * tiles * chunks) return;
    const int pair = unit / chunks, chunk = unit % chunks;
    // (long prompts first: the workgroups launched last are the short ones)
    const int t = tokens - 1 - pair / tiles, tile = pair % tiles;
    const int col = lane & 15, g = lane >> 4;
    const int head = tile * 16 + col;
    const int hq = head < heads ? head : heads - 1;           // a column pulled back inside the heads: loads are issued anyway
    const int qpos = tok_pos[t];
    const int32_t* table = page_table + (size_t)tok_seq[t] * table_width;

    LmFrag qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qf[ks].u = *reinterpret_cast<const uint4*>(q + (size_t)t * q_stride + (size_t)hq * DK + ks * 32 + 8 * g);
    lm_floatx4 o[VT];
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) o[vt] = lm_floatx4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const int key_row = 8 * (col >> 2) + (col & 3);           // the key this lane's operand row holds in the first half page

    const int page_end = chunks > 1 ? min(qpos / LM_PAGE + 1, (chunk + 1) * chunk_pages) : qpos / LM_PAGE + 1;
    for (int page = chunks > 1 ? chunk * chunk_pages : 0; page < page_end; ++page) {
        const long phys = table[page];
        const bf16_t* kp = k_pages + phys * LM_PAGE * (long)DK + (long)key_row * DK + 8 * g;
        lm_floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            LmFrag k0, k1;
            k0.u = *reinterpret_cast<const uint4*>(kp + ks * 32);
            k1.u = *reinterpret_cast<const uint4*>(kp + 4 * DK + ks * 32);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0.v, qf[ks].v, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1.v, qf[ks].v, s1, 0, 0, 0);
        }
        float s[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
        const int key0 = page * LM_PAGE + 8 * g;
        if (key0 + 7 > qpos) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (key0 + e > qpos) s[e] = -INFINITY;
        }
        float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mx = fmaxf(mx, __shfl_xor(mx, 16, RI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, RI_WAVE));
        const float m_new = fmaxf(m, mx * scale_log2);        // the scale is positive; key 0 is seen by every token: finite
        LmFrag p;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = exp2f(fmaf(s[2 * e], scale_log2, -m_new));
            const float b = exp2f(fmaf(s[2 * e + 1], scale_log2, -m_new));
            p.w[e] = pack_bf16x2(a, b);
            sum += a + b;
        }
        const float corr = exp2f(m - m_new);                  // 0 at the first page (m = -inf)
        l = l * corr + sum;
        m = m_new;
        const bf16_t* vp = v_pages + phys * (long)RANK * LM_PAGE + (long)col * LM_PAGE + 8 * g;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            LmFrag vf;
            vf.u = *reinterpret_cast<const uint4*>(vp + (long)vt * 16 * LM_PAGE);
            o[vt] *= corr;
            o[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, p.v, o[vt], 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 16, RI_WAVE);                          // a column's sum over its four lanes
    l += __shfl_xor(l, 32, RI_WAVE);
    if (chunks > 1) {
        // a chunk's share: its maximum, its sum and its sums of values as they are, for the join (a chunk without pages: -inf, 0, 0)
        if (head < heads) {
            float* pp = partial + (((size_t)t * heads + head) * chunks + chunk) * (RANK + 2);
            if (g == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
            for (int vt = 0; vt < VT; ++vt)
#pragma unroll
                for (int i = 0; i < 4; ++i) pp[2 + vt * 16 + 4 * g + i] = o[vt][i];
        }
        return;
    }
    if (sinks) l += exp2f(sinks[hq] * 1.4426950408889634f - m);
    const float inv = 1.0f / l;
    if (head < heads) {
        bf16_t* op = out + ((size_t)t * heads + head) * RANK + 4 * g;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            uint2 w;
            w.x = pack_bf16x2(o[vt][0] * inv, o[vt][1] * inv);
            w.y = pack_bf16x2(o[vt][2] * inv, o[vt][3] * inv);
            *reinterpret_cast<uint2*>(op + vt * 16) = w;
        }
    }
}

// The chunks of a token's pages, joined: the largest maximum, every chunk's sums scaled to it, the sink, the division.
__global__ void __launch_bounds__(256)
latent_attention_join_kernel(bf16_t* __restrict__ out, const float* __restrict__ partial, const float* __restrict__ sinks,
                             int heads, int chunks, int rank) {
    __shared__ float ms[LM_MAX_CHUNKS], ws[LM_MAX_CHUNKS], ls[LM_MAX_CHUNKS];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const float* pp = partial + ((size_t)t * heads + h) * chunks * (rank + 2);
    if (tid < chunks) {
        ms[tid] = pp[(size_t)tid * (rank + 2)];
        ls[tid] = pp[(size_t)tid * (rank + 2) + 1];
    }
    __syncthreads();
    float m = -INFINITY;
    for (int c = 0; c < chunks; ++c) m = fmaxf(m, ms[c]);
    if (tid < chunks) ws[tid] = exp2f(ms[tid] - m);           // a chunk's factor, once
    __syncthreads();
    float l = 0.f;
    for (int c = 0; c < chunks; ++c) l += ls[c] * ws[c];
    if (sinks) l += exp2f(sinks[h] * 1.4426950408889634f - m);
    const float inv = 1.0f / l;
    for (int d = tid; d < rank; d += 256) {
        const float* col = pp + 2 + d;
        float a = 0.f;
        int c = 0;
        for (; c + 8 <= chunks; c += 8) {                     // eight loads asked for before the first is used
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = col[(size_t)(c + i) * (rank + 2)];
#pragma unroll
            for (int i = 0; i < 8; ++i) a += v[i] * ws[c + i];
        }
        for (; c < chunks; ++c) a += col[(size_t)c * (rank + 2)] * ws[c];
        out[((size_t)t * heads + h) * rank + d] = f32_to_bf16(a * inv);
    }
}

extern "C" int ri_latent_attention_mfma_fits(int key_dim, int rank, int page_size) {
    return page_size == LM_PAGE && ((key_dim == 576 && rank == 512) || (key_dim == 288 && rank == 256) || (key_dim == 160 && rank == 128));
}

// out [tokens, heads * rank] bfloat16: causal attention of every new token's heads (q [tokens, >= heads * key_dim], the
// heads side by side) over its sequence's one key/value head of key rows of key_dim and value rows of rank.
extern "C" int ri_latent_attention_mfma(void* out, const void* q, int q_stride, const void* k_pages, const void* v_pages,
                                        const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                                        int table_width, int tokens, int heads, int key_dim, int rank, int page_size, float scale,
                                        const float* sinks, float* partial, int chunks, int chunk_pages, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && ri_latent_attention_mfma_fits(key_dim, rank, page_size),
               "latent_attention_mfma: %d tokens, %d heads, keys of %d, values of %d, pages of %d", tokens, heads, key_dim, rank, page_size);
    RI_REQUIRE(q_stride >= heads * key_dim && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)k_pages % 16 == 0 &&
               (uintptr_t)v_pages % 16 == 0 && (uintptr_t)out % 8 == 0, "latent_attention_mfma: rows of %d for %d heads of %d, or a buffer that is not aligned",
               q_stride, heads, key_dim);
    RI_REQUIRE(scale > 0.f && table_width > 0, "latent_attention_mfma: scale %g", (double)scale);
    RI_REQUIRE(chunks >= 1 && chunks <= LM_MAX_CHUNKS && (chunks == 1 || (partial && chunk_pages >= 1)) && heads <= 65535,
               "latent_attention_mfma: %d chunks of %d pages", chunks, chunk_pages);
    const int tiles = (heads + 15) / 16;
    const long pairs = (long)tokens * tiles * chunks;
    RI_REQUIRE((pairs + LM_WAVES - 1) / LM_WAVES <= 2147483647L, "latent_attention_mfma: %ld tiles exceed one launch", pairs);
    const unsigned blocks = (unsigned)((pairs + LM_WAVES - 1) / LM_WAVES);
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
#define RI_GO(KS, VT)                                                                                                   \
    latent_attention_mfma_kernel<KS, VT><<<blocks, 64 * LM_WAVES, 0, s>>>((bf16_t*)out, (const bf16_t*)q, q_stride,     \
                                                                          (const bf16_t*)k_pages, (const bf16_t*)v_pages, \
                                                                          tok_pos, tok_seq, page_table, table_width, tokens, \
                                                                          heads, tiles, scale_log2, sinks, partial, chunks, \
                                                                          chunk_pages)
    if (key_dim == 576) RI_GO(18, 32); else if (key_dim == 288) RI_GO(9, 16); else RI_GO(5, 8);
#undef RI_GO
    if (chunks > 1)
        latent_attention_join_kernel<<<dim3(tokens, heads), 256, 0, s>>>((bf16_t*)out, partial, sinks, heads, chunks, rank);
    RI_LAUNCH_CHECK("latent_attention_mfma");
    return 0;
}
