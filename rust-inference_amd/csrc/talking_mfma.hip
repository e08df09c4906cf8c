// The windowed attention whose heads talk, on the matrix cores, for prompts in bfloat16.
//
// The mixing of the heads' weights needs every head's finished softmax, so the keys are walked twice, as in the general
// kernels (talking_attention.hip), with tiles of 16 tokens of a sequence as the 16 columns of the matrix cores' tiles:
//   talking_stats_mfma:  a wavefront per (tile of tokens, head): S^T = K Q^T page by page, the distance bias, the window's
//                        mask, and each column's running maximum and sum;
//   talking_mix_mfma:    a workgroup of eight wavefronts per tile of tokens, each wavefront on an eighth of the heads:
//                        for a page it makes its heads' weights exp(s - m) / l from the first walk's numbers and leaves
//                        them in LDS (float32); after a barrier it mixes, for each of its heads, the weights of all
//                        heads (w'_h = sum_g T[h, g] w_g, on the vector units), rounds the mix to bfloat16 and adds
//                        O^T += V^T W'^T with the values of the head's own key head.
// The key rows of a half page are permuted (row r of the first half is key 8 (r / 4) + r % 4, of the second that plus
// 4), so that a lane's eight scores are eight neighbouring keys, which is how the value product wants its weights.
// Scores, the logarithm, maxima, sums, the weights before and after the mix and the accumulators are float32.  A token's
// sums run over its sequence's pages in order, whatever else the step holds.
#include "api.h"
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 tm_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float tm_floatx4;

union TmFrag {
    tm_bf16x8 v;
    uint4 u;
    uint32_t w[4];
};

#define TM_PAGE 32
#define TM_TILE 16           // tokens of a tile
#define TM_WAVES 8           // wavefronts of the second walk's workgroup

// Which tile of which sequence a workgroup takes: tiles are counted sequence after sequence.  Returns false past the last.
__device__ __forceinline__ bool tile_of(int index, const int32_t* __restrict__ cu_seqlens, int seqs, int& seq, int& first,
                                        int& count) {
    for (int s = 0; s < seqs; ++s) {
        const int n = cu_seqlens[s + 1] - cu_seqlens[s];
        const int tiles = (n + TM_TILE - 1) / TM_TILE;
        if (index < tiles) {
            seq = s;
            first = cu_seqlens[s] + index * TM_TILE;
            count = min(TM_TILE, cu_seqlens[s + 1] - first);
            return true;
        }
        index -= tiles;
    }
    return false;
}

// The eight scores of a lane (column = token, keys key0 .. key0 + 7) of head h for one page: raw products times the scale,
// minus the distance bias, minus infinity where the token does not see the key.
template <int KS>
__device__ __forceinline__ void talking_scores(float (&s)[8], const TmFrag (&qf)[KS], const bf16_t* __restrict__ kp, int dim,
                                               float scale, float b1, float b2, bool biased, int qpos, int lo, int key0) {
    tm_floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        TmFrag k0, k1;
        k0.u = *reinterpret_cast<const uint4*>(kp + ks * 32);
        k1.u = *reinterpret_cast<const uint4*>(kp + 4 * dim + ks * 32);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0.v, qf[ks].v, s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1.v, qf[ks].v, s1, 0, 0, 0);
    }
    const float raw[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int key = key0 + e;
        float v = raw[e] * scale;
        if (biased) v -= b1 * log1pf(b2 * (float)max(qpos - key, 0));
        s[e] = (key > qpos || key < lo) ? -INFINITY : v;
    }
}

template <int KS>
__global__ void __launch_bounds__(64)
talking_stats_mfma_kernel(float* __restrict__ stats, const bf16_t* __restrict__ q, int q_stride, int q_off,
                          const bf16_t* __restrict__ k_pages, const int32_t* __restrict__ tok_pos,
                          const int32_t* __restrict__ cu_seqlens, int seqs, const int32_t* __restrict__ page_table,
                          int table_width, int heads, int kv_heads, int window, float scale, const float* __restrict__ r1,
                          const float* __restrict__ r2) {
    constexpr int DIM = 32 * KS;
    int seq, first, count;
    if (!tile_of(blockIdx.x, cu_seqlens, seqs, seq, first, count)) return;
    const int h = blockIdx.y, lane = threadIdx.x;
    const int col = lane & 15, g = lane >> 4;
    const int t = first + min(col, count - 1);                 // a column pulled back inside the tile: loads are issued anyway
    const int qpos = tok_pos[t];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int kvh = h / (heads / kv_heads);
    const int32_t* table = page_table + (size_t)seq * table_width;
    TmFrag qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qf[ks].u = *reinterpret_cast<const uint4*>(q + (size_t)t * q_stride + q_off + (size_t)h * DIM + ks * 32 + 8 * g);
    const bool biased = r1 != nullptr;
    const float b1 = biased ? r1[h] : 0.f, b2 = biased ? r2[h] : 0.f;
    const int pos_first = tok_pos[first], pos_last = pos_first + count - 1;
    const int lo_first = window > 0 ? max(0, pos_first - window + 1) : 0;
    const int key_row = 8 * (col >> 2) + (col & 3);
    float m = -INFINITY, l = 0.f;
    for (int page = lo_first / TM_PAGE; page <= pos_last / TM_PAGE; ++page) {
        const bf16_t* kp = k_pages + (((long)table[page] * kv_heads + kvh) * TM_PAGE + key_row) * (long)DIM + 8 * g;
        float s[8];
        talking_scores<KS>(s, qf, kp, DIM, scale, b1, b2, biased, qpos, lo, page * TM_PAGE + 8 * g);
        float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mx = fmaxf(mx, __shfl_xor(mx, 16, RI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, RI_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // a column that has seen no key yet
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += expf(s[e] - m_safe);
        l = l * expf(m - m_safe) + sum;                          // the factor is 0 while m is -inf
        m = m_new;
    }
    l += __shfl_xor(l, 16, RI_WAVE);
    l += __shfl_xor(l, 32, RI_WAVE);
    if (g == 0 && col < count) {
        stats[((size_t)t * heads + h) * 2] = m;
        stats[((size_t)t * heads + h) * 2 + 1] = l;
    }
}

template <int KS, int HPW>
__global__ void __launch_bounds__(64 * TM_WAVES)
talking_mix_mfma_kernel(bf16_t* __restrict__ out, const float* __restrict__ stats, const bf16_t* __restrict__ q, int q_stride,
                        int q_off, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ cu_seqlens, int seqs,
                        const int32_t* __restrict__ page_table, int table_width, int kv_heads, int window, float scale,
                        const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ talk) {
    constexpr int DIM = 32 * KS, VT = DIM / 16, HEADS = HPW * TM_WAVES;
    extern __shared__ float lds[];
    float* ps = lds;                                           // [HEADS][TM_TILE][TM_PAGE] the heads' weights of a page
    float* tk = ps + HEADS * TM_TILE * TM_PAGE;                // [HEADS][HEADS] the mixing matrix
    int seq, first, count;
    if (!tile_of(blockIdx.x, cu_seqlens, seqs, seq, first, count)) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, g = lane >> 4;
    const int t = first + min(col, count - 1);
    const int qpos = tok_pos[t];
    const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int share = HEADS / kv_heads;
    const int32_t* table = page_table + (size_t)seq * table_width;
    for (int e = threadIdx.x; e < HEADS * HEADS; e += 64 * TM_WAVES) tk[e] = talk ? talk[e] : (e / HEADS == e % HEADS ? 1.f : 0.f);
    const bool biased = r1 != nullptr;
    float ms[HPW], inv_l[HPW], b1[HPW], b2[HPW];
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        const int h = wave * HPW + i;
        ms[i] = stats[((size_t)t * HEADS + h) * 2];
        inv_l[i] = 1.0f / stats[((size_t)t * HEADS + h) * 2 + 1];
        b1[i] = biased ? r1[h] : 0.f;
        b2[i] = biased ? r2[h] : 0.f;
    }
    tm_floatx4 o[HPW][VT];
#pragma unroll
    for (int i = 0; i < HPW; ++i)
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) o[i][vt] = tm_floatx4{0.f, 0.f, 0.f, 0.f};
    const int pos_first = tok_pos[first], pos_last = pos_first + count - 1;
    const int lo_first = window > 0 ? max(0, pos_first - window + 1) : 0;
    const int key_row = 8 * (col >> 2) + (col & 3);
    __syncthreads();
    for (int page = lo_first / TM_PAGE; page <= pos_last / TM_PAGE; ++page) {
        const long phys = table[page];
        // this wavefront's heads: their weights of the page, into LDS
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int h = wave * HPW + i;
            const bf16_t* kp = k_pages + ((phys * kv_heads + h / share) * TM_PAGE + key_row) * (long)DIM + 8 * g;
            TmFrag qf[KS];                                     // (fetched again a page: the caches hold them, the registers are the sums')
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                qf[ks].u = *reinterpret_cast<const uint4*>(q + (size_t)t * q_stride + q_off + (size_t)h * DIM + ks * 32 + 8 * g);
            float s[8];
            talking_scores<KS>(s, qf, kp, DIM, scale, b1[i], b2[i], biased, qpos, lo, page * TM_PAGE + 8 * g);
            float4 lo4, hi4;
            lo4.x = expf(s[0] - ms[i]) * inv_l[i]; lo4.y = expf(s[1] - ms[i]) * inv_l[i];
            lo4.z = expf(s[2] - ms[i]) * inv_l[i]; lo4.w = expf(s[3] - ms[i]) * inv_l[i];
            hi4.x = expf(s[4] - ms[i]) * inv_l[i]; hi4.y = expf(s[5] - ms[i]) * inv_l[i];
            hi4.z = expf(s[6] - ms[i]) * inv_l[i]; hi4.w = expf(s[7] - ms[i]) * inv_l[i];
            float* pp = ps + ((size_t)h * TM_TILE + col) * TM_PAGE + 8 * g;
            *reinterpret_cast<float4*>(pp) = lo4;
            *reinterpret_cast<float4*>(pp + 4) = hi4;
        }
        __syncthreads();
        // the mix for this wavefront's heads, then their value products
        float mixed[HPW][8];
#pragma unroll
        for (int i = 0; i < HPW; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) mixed[i][e] = 0.f;
        for (int gh = 0; gh < HEADS; ++gh) {
            const float* pp = ps + ((size_t)gh * TM_TILE + col) * TM_PAGE + 8 * g;
            const float4 a = *reinterpret_cast<const float4*>(pp), b = *reinterpret_cast<const float4*>(pp + 4);
            const float w8[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int i = 0; i < HPW; ++i) {
                const float c = tk[(wave * HPW + i) * HEADS + gh];
#pragma unroll
                for (int e = 0; e < 8; ++e) mixed[i][e] += c * w8[e];
            }
        }
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int h = wave * HPW + i;
            TmFrag p;
#pragma unroll
            for (int e = 0; e < 4; ++e) p.w[e] = pack_bf16x2(mixed[i][2 * e], mixed[i][2 * e + 1]);
            const bf16_t* vp = v_pages + ((phys * kv_heads + h / share) * (long)DIM + col) * TM_PAGE + 8 * g;
#pragma unroll
            for (int vt = 0; vt < VT; ++vt) {
                TmFrag vf;
                vf.u = *reinterpret_cast<const uint4*>(vp + (long)vt * 16 * TM_PAGE);
                o[i][vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, p.v, o[i][vt], 0, 0, 0);
            }
        }
        __syncthreads();                                       // before the next page's weights overwrite these
    }
    if (col < count) {
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            bf16_t* op = out + (size_t)t * HEADS * DIM + (size_t)(wave * HPW + i) * DIM + 4 * g;
#pragma unroll
            for (int vt = 0; vt < VT; ++vt) {
                uint2 w;
                w.x = pack_bf16x2(o[i][vt][0], o[i][vt][1]);
                w.y = pack_bf16x2(o[i][vt][2], o[i][vt][3]);
                *reinterpret_cast<uint2*>(op + vt * 16) = w;
            }
        }
    }
}

extern "C" int ri_talking_attention_mfma_fits(int heads, int kv_heads, int dim, int page_size) {
    return page_size == TM_PAGE && (dim == 32 || dim == 64 || dim == 128) && heads % TM_WAVES == 0 && heads / TM_WAVES <= 4 &&
           kv_heads >= 1 && heads % kv_heads == 0;
}

// out [tokens, heads * dim] bfloat16; stats: float32 workspace [tokens][heads][2]; tiles: an upper bound on the tiles of
// 16 tokens that the sequences' new tokens make (every sequence's count rounded up).
extern "C" int ri_talking_attention_mfma(void* out, float* stats, const void* q, int q_stride, int q_off, const void* k_pages,
                                         const void* v_pages, const int32_t* tok_pos, const int32_t* cu_seqlens, int seqs,
                                         const int32_t* page_table, int table_width, int tiles, int heads, int kv_heads, int dim,
                                         int page_size, int window, float scale, const float* r1, const float* r2,
                                         const float* talk, void* stream) {
    RI_REQUIRE(seqs > 0 && tiles > 0 && ri_talking_attention_mfma_fits(heads, kv_heads, dim, page_size),
               "talking_attention_mfma: %d sequences, %d heads over %d of %d, pages of %d", seqs, heads, kv_heads, dim, page_size);
    RI_REQUIRE(q_off >= 0 && q_off + heads * dim <= q_stride && q_stride % 8 == 0 && q_off % 8 == 0 && (uintptr_t)q % 16 == 0 &&
               (uintptr_t)k_pages % 16 == 0 && (uintptr_t)v_pages % 16 == 0 && (uintptr_t)out % 8 == 0,
               "talking_attention_mfma: column %d of rows of %d, or a buffer that is not aligned", q_off, q_stride);
    RI_REQUIRE((r1 == nullptr) == (r2 == nullptr) && window >= 0 && table_width > 0 && stats, "talking_attention_mfma: arguments");
    const size_t lds = ((size_t)heads * TM_TILE * TM_PAGE + (size_t)heads * heads) * sizeof(float);
    RI_REQUIRE(lds <= 64 * 1024 + 4096, "talking_attention_mfma: %d heads need %zu bytes of LDS", heads, lds);
    hipStream_t s = (hipStream_t)stream;
    const int hpw = heads / TM_WAVES;
#define RI_STATS(KS)                                                                                                    \
    talking_stats_mfma_kernel<KS><<<dim3(tiles, heads), 64, 0, s>>>(stats, (const bf16_t*)q, q_stride, q_off,          \
                                                                     (const bf16_t*)k_pages, tok_pos, cu_seqlens, seqs, \
                                                                     page_table, table_width, heads, kv_heads, window, scale, r1, r2)
#define RI_MIX(KS, HPW)                                                                                                 \
    do {                                                                                                                \
        if (lds > 64 * 1024)                                                                                            \
            hipFuncSetAttribute((const void*)talking_mix_mfma_kernel<KS, HPW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
        talking_mix_mfma_kernel<KS, HPW><<<tiles, 64 * TM_WAVES, lds, s>>>(                                             \
            (bf16_t*)out, stats, (const bf16_t*)q, q_stride, q_off, (const bf16_t*)k_pages, (const bf16_t*)v_pages, tok_pos, \
            cu_seqlens, seqs, page_table, table_width, kv_heads, window, scale, r1, r2, talk);                          \
    } while (0)
#define RI_BY_HEADS(KS)                                                                                                 \
    do {                                                                                                                \
        RI_STATS(KS);                                                                                                   \
        if (hpw == 1) RI_MIX(KS, 1); else if (hpw == 2) RI_MIX(KS, 2); else if (hpw == 3) RI_MIX(KS, 3); else RI_MIX(KS, 4); \
    } while (0)
    if (dim == 32) RI_BY_HEADS(1); else if (dim == 64) RI_BY_HEADS(2); else RI_BY_HEADS(4);
#undef RI_BY_HEADS
#undef RI_MIX
#undef RI_STATS
    RI_LAUNCH_CHECK("talking_attention_mfma");
    return 0;
}
