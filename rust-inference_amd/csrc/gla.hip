// Gated linear attention: a state of dim x vdim numbers per head and sequence instead of keys and values,
//     S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t,
// with one decay per key channel, alpha = sigmoid(z)^(1/tau) = exp(log_sigmoid(z) / tau).  State, decay, its
// logarithm and exponential, and the sums are float32; q, k, v and z come from products.
//
// The scan walks a sequence's tokens in order; what runs side by side is everything else: a workgroup owns one
// (sequence, head) and GLA_COLS columns of the state, its 256 threads as 16 columns x 16 slices of rows, every
// thread keeping its rows of its column (slice r: rows r * rpt .. r * rpt + rpt - 1, rpt = ceil(dim / 16); read
// from LDS 16 bytes at a time where rpt is a multiple of 4) in registers.  For prompts the decays are made by a
// pass of their own over all tokens at once (gla_decay_kernel), so that no logarithm stands in the walk.  Tokens go through in blocks of nb: a block's q, k, alpha
// and v are staged in LDS (two buffers), the next block's loads are asked for before the block in work is
// computed and stored after it, so memory's latency is paid once a block and behind the arithmetic; the 16
// slices' shares of o_t meet through a shuffle inside a wavefront and through LDS between the four wavefronts,
// with one barrier a block.  The same kernel serves a step of one token.
#include "api.h"
#include "common.h"

#define GLA_COLS 16
#define GLA_SLICES 16
#define GLA_MAX_ROWS 32          // rows of a column per thread: dim <= 16 * 32
#define GLA_MAX_NB 32            // tokens of a block
#define GLA_STAGE 16             // most staged elements of q, k and z per thread and block: nb * dim <= 16 * 256 (STAGE: 4 or 16)
#define GLA_VSTAGE (GLA_MAX_NB * GLA_COLS / 256)

__device__ __forceinline__ float log_sigmoid(float z) {
    // min(z, 0) - log(1 + exp(-|z|)): no overflow on either side
    return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

// z <- exp(log_sigmoid(z + bias) / tau) in place, for all tokens at once.
__global__ void gla_decay_kernel(float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau, long total,
                                 int width) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    z[e] = expf(log_sigmoid(z[e] + (z_bias ? z_bias[e % width] : 0.f)) * inv_tau);
}

// FIXED: the decay is one constant per head (head_decay[h]) instead of a number per token and key channel, and q, k
// and v pass through silu on their way in (linear attention with a fixed decay); z is then not read.
__device__ __forceinline__ float silu_of(float v) { return v / (1.0f + expf(-v)); }

template <typename TA, int RPT, int STAGE, bool FIXED>
__global__ void __launch_bounds__(256)
gla_scan_kernel(float* __restrict__ out, const TA* __restrict__ proj, int row, int q_off, int k_off, int v_off,
                const float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau, float q_scale,
                float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots,
                int heads, int dim, int vdim, int nb, int z_is_decay, const float* __restrict__ head_decay) {
    extern __shared__ float lds[];                           // two buffers of nb tokens: q, k, alpha (dim each), v (16)
    __shared__ float part[2][GLA_MAX_NB][4][GLA_COLS];       // the wavefronts' shares of o_t, two blocks in flight
    const int b = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * GLA_COLS;
    const int tid = threadIdx.x, c = tid % GLA_COLS, r = tid / GLA_COLS, wave = tid / RI_WAVE;
    const int col = col0 + c;
    const bool live = col < vdim;
    const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
    if (t1 <= t0) return;
    const int stride = 3 * dim + GLA_COLS, per = nb * dim;
    float* S = state + (((size_t)slots[b] * heads + h) * dim) * vdim + col;
    const int rpt = (dim + GLA_SLICES - 1) / GLA_SLICES, row0 = r * rpt;   // this thread's rows: row0 .. row0 + rpt - 1
    const int rows_here = max(0, min(rpt, dim - row0));
    float s[GLA_MAX_ROWS];
#pragma unroll
    for (int j = 0; j < GLA_MAX_ROWS; ++j) s[j] = (live && j < rows_here) ? S[(size_t)(row0 + j) * vdim] : 0.f;

    // a block's inputs on their way: every load is issued whatever the indices are, from a token and a column
    // pulled back inside the data
    float rq[STAGE], rk[STAGE], rz[STAGE], rv[GLA_VSTAGE];
    // which token of a block and which channel each staged element is: the same for every block, worked out once
    // (a division a token would cost more than the token's arithmetic)
    int s_tok[STAGE], s_ch[STAGE], v_tok[GLA_VSTAGE], v_col[GLA_VSTAGE];
#pragma unroll
    for (int j = 0; j < STAGE; ++j) {
        const int e = min(tid + j * 256, per - 1);
        s_tok[j] = e / dim;
        s_ch[j] = e - s_tok[j] * dim;
    }
#pragma unroll
    for (int j = 0; j < GLA_VSTAGE; ++j) {
        const int e = min(tid + j * 256, nb * GLA_COLS - 1);
        v_tok[j] = e / GLA_COLS;
        v_col[j] = min(col0 + e % GLA_COLS, vdim - 1);
    }
    auto ask = [&](int tb) {
#pragma unroll
        for (int j = 0; j < STAGE; ++j) {
            if (j * 256 >= per) break;                       // (per is the same for all: no thread has an element here)
            const int tok = min(tb + s_tok[j], t1 - 1), i = s_ch[j];
            const TA* x = proj + (size_t)tok * row + h * dim + i;
            rq[j] = to_f32(x[q_off]);
            rk[j] = to_f32(x[k_off]);
            if (!FIXED) rz[j] = z[((size_t)tok * heads + h) * dim + i];
        }
#pragma unroll
        for (int j = 0; j < GLA_VSTAGE; ++j) {
            if (j * 256 >= nb * GLA_COLS) break;
            const int tok = min(tb + v_tok[j], t1 - 1);
            rv[j] = to_f32(proj[(size_t)tok * row + v_off + h * vdim + v_col[j]]);
        }
    };
    auto put = [&](int which) {
        float* buf = lds + (size_t)which * nb * stride;
#pragma unroll
        for (int j = 0; j < STAGE; ++j) {
            if (j * 256 >= per) break;
            if (tid + j * 256 < per) {
                const int i = s_ch[j];
                float* at = buf + (size_t)s_tok[j] * stride;
                if (FIXED) {
                    at[i] = silu_of(rq[j]) * q_scale;
                    at[dim + i] = silu_of(rk[j]);
                    at[2 * dim + i] = head_decay[h];
                } else {
                    at[i] = rq[j] * q_scale;
                    at[dim + i] = rk[j];
                    at[2 * dim + i] = z_is_decay ? rz[j] : expf(log_sigmoid(rz[j] + (z_bias ? z_bias[h * dim + i] : 0.f)) * inv_tau);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < GLA_VSTAGE; ++j) {
            const int e = tid + j * 256;
            if (e < nb * GLA_COLS) buf[(size_t)v_tok[j] * stride + 3 * dim + e % GLA_COLS] = FIXED ? silu_of(rv[j]) : rv[j];
        }
    };
    ask(t0);
    put(0);
    __syncthreads();
    int blk = 0;
    for (int tb = t0; tb < t1; tb += nb, ++blk) {
        const bool more = tb + nb < t1;                      // the same for the whole workgroup
        if (more) ask(tb + nb);
        const float* buf = lds + (size_t)(blk & 1) * nb * stride;
        // eight tokens at a time: their state updates follow one another, but nothing else of a token waits for
        // the token before, so the LDS reads run ahead and the slices' shares meet (two shuffles a token) after the
        // eight, side by side (a workgroup's four wavefronts are one a SIMD: nothing else hides a latency here)
        auto token = [&](const float* at) -> float {
            const float v = at[3 * dim + c];
            float o = 0.f;
            if (RPT > 0) {                                   // dim = 16 RPT, RPT a multiple of 4: 16 bytes a read, no guards
#pragma unroll
                for (int j = 0; j < (RPT > 0 ? RPT : 4); j += 4) {
                    {
                        const float4 q4 = *reinterpret_cast<const float4*>(at + row0 + j);
                        const float4 k4 = *reinterpret_cast<const float4*>(at + dim + row0 + j);
                        const float4 a4 = *reinterpret_cast<const float4*>(at + 2 * dim + row0 + j);
                        s[j] = a4.x * s[j] + k4.x * v;
                        s[j + 1] = a4.y * s[j + 1] + k4.y * v;
                        s[j + 2] = a4.z * s[j + 2] + k4.z * v;
                        s[j + 3] = a4.w * s[j + 3] + k4.w * v;
                        o += (s[j] * q4.x + s[j + 1] * q4.y) + (s[j + 2] * q4.z + s[j + 3] * q4.w);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < GLA_MAX_ROWS; ++j) {
                    if (j < rows_here) {
                        const int i = row0 + j;
                        s[j] = at[2 * dim + i] * s[j] + at[dim + i] * v;
                        o += s[j] * at[i];
                    }
                }
            }
            return o;
        };
        for (int n0 = 0; n0 < nb; n0 += 8) {
            if (tb + n0 >= t1) break;                        // the same for the whole workgroup
            float oo[8];
            if (n0 + 8 <= nb && tb + n0 + 8 <= t1) {
#pragma unroll
                for (int u = 0; u < 8; ++u) oo[u] = token(buf + (size_t)(n0 + u) * stride);
            } else {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    oo[u] = 0.f;
                    if (n0 + u < nb && tb + n0 + u < t1) oo[u] = token(buf + (size_t)(n0 + u) * stride);
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {                    // lanes of a wavefront: 4 slices x 16 columns
                oo[u] += __shfl_xor(oo[u], 16, RI_WAVE);
                oo[u] += __shfl_xor(oo[u], 32, RI_WAVE);
            }
            if ((tid & (RI_WAVE - 1)) < GLA_COLS) {
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (n0 + u < nb) part[blk & 1][n0 + u][wave][c] = oo[u];
            }
        }
        if (more) put((blk + 1) & 1);
        __syncthreads();
        for (int e = tid; e < nb * GLA_COLS; e += 256) {
            const int n = e / GLA_COLS, cc = e % GLA_COLS;
            if (tb + n < t1 && col0 + cc < vdim) {
                const float (*p)[GLA_COLS] = part[blk & 1][n];
                out[((size_t)(tb + n) * heads + h) * vdim + col0 + cc] = ((p[0][cc] + p[1][cc]) + p[2][cc]) + p[3][cc];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < GLA_MAX_ROWS; ++j)
        if (live && j < rows_here) S[(size_t)(row0 + j) * vdim] = s[j];
}

static int gla_scan_go(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                       float* z, const float* z_bias, float tau, float q_scale, float* state,
                       const int32_t* cu_seqlens, const int32_t* slots, int seqs, int tokens, int heads, int dim,
                       int vdim, const float* head_decay, void* stream) {
    RI_REQUIRE(seqs > 0 && tokens >= seqs && heads > 0 && dim > 0 && vdim > 0, "gla_scan: %d sequences, %d heads of %d x %d", seqs, heads, dim, vdim);
    RI_REQUIRE(dim <= GLA_SLICES * GLA_MAX_ROWS, "gla_scan: key heads of %d exceed the kernel's %d", dim, GLA_SLICES * GLA_MAX_ROWS);
    RI_REQUIRE(heads <= 65535 && seqs <= 65535, "gla_scan: %d heads of %d sequences exceed one launch", heads, seqs);
    RI_REQUIRE(tau > 0.f, "gla_scan: tau %g must be positive", (double)tau);
    RI_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + heads * dim <= row && k_off + heads * dim <= row &&
               v_off + heads * vdim <= row, "gla_scan: q, k, v at %d, %d, %d do not fit rows of %d", q_off, k_off, v_off, row);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "gla_scan: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((vdim + GLA_COLS - 1) / GLA_COLS, heads, seqs);
    // tokens a block: as many as the staging registers hold (dim <= 512: at least eight), at most 32; 16 and 8
    // where the workgroups outnumber the compute units, so that several fit one unit's LDS and hide one another's
    // waits; a step of single tokens 1
    int nb = GLA_STAGE * 256 / dim;
    nb = nb > GLA_MAX_NB ? GLA_MAX_NB : nb;
    const long wgs = (long)grid.x * grid.y * grid.z, cus = ri_compute_units();
    if (nb > 16 && wgs > cus) nb = 16;
    if (nb > 8 && wgs > 3 * cus) nb = 8;
    if (tokens == seqs) nb = 1;
    const size_t lds = (size_t)2 * nb * (3 * dim + GLA_COLS) * sizeof(float);
    // a prompt: the decays of all its tokens in one pass, in place of z, before the walk
    int z_is_decay = 0;
    if (tokens > seqs && !head_decay) {
        const long total = (long)tokens * heads * dim;
        RI_REQUIRE((total + 255) / 256 <= 2147483647L, "gla_scan: %ld decays exceed one launch", total);
        gla_decay_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(z, z_bias, 1.0f / tau, total, heads * dim);
        z_is_decay = 1;
    }
    // key heads of 64, 128, 256 or 512: a thread's rows are a fixed number, a multiple of 4, read 16 bytes at a time
    const int fixed = (dim == 64 || dim == 128 || dim == 256 || dim == 512) ? dim / GLA_SLICES : 0;
    // (more than 64 KB of dynamic LDS has to be asked for, once for every form of the kernel)
#define RI_GLA_GO(T, V, G, F)                                                                                        \
    if (lds > 48 * 1024) {                                                                                           \
        static bool asked = false;                                                                                   \
        if (!asked) {                                                                                                \
            hipError_t e_ = hipFuncSetAttribute((const void*)gla_scan_kernel<T, V, G, F>,                             \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);             \
            RI_REQUIRE(e_ == hipSuccess, "gla_scan: %s", hipGetErrorString(e_));                                     \
            asked = true;                                                                                            \
        }                                                                                                            \
    }                                                                                                                \
    gla_scan_kernel<T, V, G, F><<<grid, 256, lds, s>>>(out, (const T*)proj, row, q_off, k_off, v_off, z, z_bias, 1.0f / tau,\
                                                 q_scale, state, cu_seqlens, slots, heads, dim, vdim, nb, z_is_decay, head_decay)
    // (blocks of up to 4 * 256 staged elements run with a quarter of the staging registers: more wavefronts a SIMD)
    const bool few = (long)nb * dim <= 4 * 256;
#define RI_GLA_STAGE(T, R)                                                                                           \
    if (head_decay) { if (few) { RI_GLA_GO(T, R, 4, true); } else { RI_GLA_GO(T, R, 16, true); } }                    \
    else            { if (few) { RI_GLA_GO(T, R, 4, false); } else { RI_GLA_GO(T, R, 16, false); } }
#define RI_GLA_ROWS(T)                                                                                               \
    switch (fixed) {                                                                                                 \
        case 4: RI_GLA_STAGE(T, 4) break;                                                                            \
        case 8: RI_GLA_STAGE(T, 8) break;                                                                            \
        case 16: RI_GLA_STAGE(T, 16) break;                                                                          \
        case 32: RI_GLA_STAGE(T, 32) break;                                                                          \
        default: RI_GLA_STAGE(T, 0) break;                                                                           \
    }
    if (act_dtype == RI_F32) { RI_GLA_ROWS(float) } else { RI_GLA_ROWS(bf16_t) }
#undef RI_GLA_ROWS
#undef RI_GLA_STAGE
#undef RI_GLA_GO
    RI_LAUNCH_CHECK("gla_scan");
    return 0;
}

extern "C" int ri_gla_scan(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                           float* z, const float* z_bias, float tau, float q_scale, float* state,
                           const int32_t* cu_seqlens, const int32_t* slots, int seqs, int tokens, int heads, int dim,
                           int vdim, void* stream) {
    RI_REQUIRE(z, "gla_scan: no decay logits");
    return gla_scan_go(out, proj, act_dtype, row, q_off, k_off, v_off, z, z_bias, tau, q_scale, state, cu_seqlens, slots,
                       seqs, tokens, heads, dim, vdim, nullptr, stream);
}

// Linear attention with one fixed decay per head: S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with
// q = silu(.) * q_scale, k = silu(.), v = silu(.) of the projection's columns; head_decay: float32 [heads].
extern "C" int ri_decay_scan(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                             const float* head_decay, float q_scale, float* state, const int32_t* cu_seqlens,
                             const int32_t* slots, int seqs, int tokens, int heads, int dim, int vdim, void* stream) {
    RI_REQUIRE(head_decay, "decay_scan: no decays");
    return gla_scan_go(out, proj, act_dtype, row, q_off, k_off, v_off, nullptr, nullptr, 1.0f, q_scale, state, cu_seqlens,
                       slots, seqs, tokens, heads, dim, vdim, head_decay, stream);
}

// The scan's result per head through an RMS norm over vdim (one gain for all heads) and times silu(gate):
// one wavefront per (token, head).
#define GLA_NORM_PER_LANE 8      // vdim <= 64 * 8

template <typename TA>
__global__ void gla_norm_gate_kernel(TA* __restrict__ out, const float* __restrict__ o, const TA* __restrict__ proj,
                                     int row, int g_off, const float* __restrict__ gain, float eps, long items,
                                     int heads, int vdim) {
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const long item = (long)blockIdx.x * (blockDim.x / RI_WAVE) + threadIdx.x / RI_WAVE;
    if (item >= items) return;
    const long t = item / heads;
    const int h = (int)(item % heads);
    const float* x = o + (size_t)item * vdim;
    const TA* g = proj + (size_t)t * row + g_off + (size_t)h * vdim;
    float v[GLA_NORM_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < GLA_NORM_PER_LANE; ++j) {
        const int i = lane + j * RI_WAVE;
        v[j] = i < vdim ? x[i] : 0.f;
        ss += v[j] * v[j];
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
#pragma unroll
    for (int j = 0; j < GLA_NORM_PER_LANE; ++j) {
        const int i = lane + j * RI_WAVE;
        if (i >= vdim) continue;
        const float gate = to_f32(g[i]);
        from_f32(out + (size_t)item * vdim + i, v[j] * inv * gain[i] * (gate / (1.0f + expf(-gate))));
    }
}

// The same 16 bytes a lane, for value heads of 8 lanes' worth of eight elements or a power-of-two fraction (vdim 8,
// 16, ... 512): vdim / 8 lanes make a head, a wavefront works on 512 / vdim heads at once.
template <typename TA>
__global__ void __launch_bounds__(256)
gla_norm_gate_vec_kernel(TA* __restrict__ out, const float* __restrict__ o, const TA* __restrict__ proj, int row, int g_off,
                         const float* __restrict__ gain, float eps, long items, int heads, int vdim) {
    const int lanes_per_head = vdim / 8;
    const int heads_at_once = RI_WAVE / lanes_per_head;
    const int lane = threadIdx.x & (RI_WAVE - 1);
    const long wave_id = (long)blockIdx.x * (blockDim.x / RI_WAVE) + threadIdx.x / RI_WAVE;
    const long item = wave_id * heads_at_once + lane / lanes_per_head;
    const int piece = lane % lanes_per_head;
    if (item >= items) return;                               // lanes of a head leave together
    const long t = item / heads;
    const int h = (int)(item % heads);
    const float* x = o + (size_t)item * vdim + piece * 8;
    const float4 a = *reinterpret_cast<const float4*>(x), b = *reinterpret_cast<const float4*>(x + 4);
    float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float gate[8];
    const TA* g = proj + (size_t)t * row + g_off + (size_t)h * vdim + piece * 8;
    if (sizeof(TA) == 2) {
        const uint4 w = *reinterpret_cast<const uint4*>(g);
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            gate[2 * i] = __uint_as_float(ww[i] << 16);
            gate[2 * i + 1] = __uint_as_float(ww[i] & 0xFFFF0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) gate[i] = to_f32(g[i]);
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
    for (int m = lanes_per_head / 2; m > 0; m >>= 1) ss += __shfl_xor(ss, m, RI_WAVE);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
    const float4 ga = *reinterpret_cast<const float4*>(gain + piece * 8), gb = *reinterpret_cast<const float4*>(gain + piece * 8 + 4);
    const float gn[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
    float r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = v[e] * inv * gn[e] * (gate[e] / (1.0f + expf(-gate[e])));
    TA* dst = out + (size_t)item * vdim + piece * 8;
    if (sizeof(TA) == 2) {
        *reinterpret_cast<uint4*>(dst) = make_uint4(pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3]), pack_bf16x2(r[4], r[5]),
                                                    pack_bf16x2(r[6], r[7]));
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) from_f32(dst + e, r[e]);
    }
}

extern "C" int ri_gla_norm_gate(void* out, const float* o, const void* proj, int act_dtype, int row, int g_off,
                                const float* gain, float eps, int tokens, int heads, int vdim, void* stream) {
    RI_REQUIRE(tokens > 0 && heads > 0 && vdim > 0 && vdim <= RI_WAVE * GLA_NORM_PER_LANE,
               "gla_norm_gate: %d tokens, %d heads of %d", tokens, heads, vdim);
    RI_REQUIRE(g_off >= 0 && g_off + heads * vdim <= row, "gla_norm_gate: the gate at %d does not fit rows of %d", g_off, row);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "gla_norm_gate: dtype %d", act_dtype);
    const long items = (long)tokens * heads;
    const long blocks = (items + 3) / 4;
    RI_REQUIRE(blocks <= 2147483647L, "gla_norm_gate: %ld heads exceed one launch", items);
    hipStream_t s = (hipStream_t)stream;
    const int lph = vdim / 8;
    if (vdim % 8 == 0 && lph <= 64 && (lph & (lph - 1)) == 0 && row % 8 == 0 && g_off % 8 == 0) {
        const long waves = (items + (64 / lph) - 1) / (64 / lph), vblocks = (waves + 3) / 4;
        if (act_dtype == RI_F32)
            gla_norm_gate_vec_kernel<float><<<(unsigned)vblocks, 256, 0, s>>>((float*)out, o, (const float*)proj, row, g_off,
                                                                              gain, eps, items, heads, vdim);
        else
            gla_norm_gate_vec_kernel<bf16_t><<<(unsigned)vblocks, 256, 0, s>>>((bf16_t*)out, o, (const bf16_t*)proj, row,
                                                                               g_off, gain, eps, items, heads, vdim);
        RI_LAUNCH_CHECK("gla_norm_gate");
        return 0;
    }
    if (act_dtype == RI_F32)
        gla_norm_gate_kernel<float><<<(unsigned)blocks, 256, 0, s>>>((float*)out, o, (const float*)proj, row, g_off, gain, eps,
                                                                     items, heads, vdim);
    else
        gla_norm_gate_kernel<bf16_t><<<(unsigned)blocks, 256, 0, s>>>((bf16_t*)out, o, (const bf16_t*)proj, row, g_off, gain,
                                                                      eps, items, heads, vdim);
    RI_LAUNCH_CHECK("gla_norm_gate");
    return 0;
}

// ------------------------------------------------------------------ one new token a sequence
// The recurrence's step, the norm and the gate in one kernel: a workgroup owns one (sequence, head) and the whole
// state of it, vdim / 4 groups of four columns x 256 / (vdim / 4) slices of rows, every thread's piece of the
// state asked for up front in 16-byte loads (a step's time is the state's trip from memory and back), updated
// in registers and stored; the slices' shares of o meet in LDS, where the head is normed and gated.
#define GLA_STEP_ROWS 32

// FIXED (linear attention with one decay per head, head_decay[h]): q, k and v pass through silu, z is not read, and the
// step's result leaves as it is, float32 in raw[seqs][heads * vdim]: its norm runs over all heads together, afterwards.
template <typename TA, int ROWS, bool FIXED>
__global__ void __launch_bounds__(256)
gla_step_kernel(TA* __restrict__ out, const TA* __restrict__ proj, int row, int q_off, int k_off, int v_off, int g_off,
                const float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau, float q_scale,
                float* __restrict__ state, const int32_t* __restrict__ slots, const float* __restrict__ gain, float eps,
                int heads, int dim, int vdim, int groups, int slices, const float* __restrict__ head_decay,
                float* __restrict__ raw) {
    __shared__ float qs[GLA_SLICES * GLA_MAX_ROWS], ks[GLA_SLICES * GLA_MAX_ROWS], as[GLA_SLICES * GLA_MAX_ROWS];
    __shared__ __attribute__((aligned(16))) float red[1024];                 // [slices][vdim]
    __shared__ float scratch[16];
    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int g = tid % groups, r = tid / groups;
    const int rpt = (dim + slices - 1) / slices, row0 = r * rpt;
    const int rows_here = r < slices ? max(0, min(rpt, dim - row0)) : 0;
    float* S = state + (((size_t)slots[b] * heads + h) * dim) * vdim + 4 * g;
    float4 s[ROWS];                                         // ROWS: 8, 16 or 32, the least that holds a slice
#pragma unroll
    for (int j = 0; j < ROWS; ++j)                           // every load issued, from a row pulled back inside the state
        s[j] = *reinterpret_cast<const float4*>(S + (size_t)min(row0 + j, dim - 1) * vdim);
    const TA* x = proj + (size_t)b * row;
    for (int i = tid; i < dim; i += 256) {
        if (FIXED) {
            qs[i] = silu_of(to_f32(x[q_off + h * dim + i])) * q_scale;
            ks[i] = silu_of(to_f32(x[k_off + h * dim + i]));
            as[i] = head_decay[h];
        } else {
            qs[i] = to_f32(x[q_off + h * dim + i]) * q_scale;
            ks[i] = to_f32(x[k_off + h * dim + i]);
            as[i] = expf(log_sigmoid(z[((size_t)b * heads + h) * dim + i] + (z_bias ? z_bias[h * dim + i] : 0.f)) * inv_tau);
        }
    }
    const TA* vx = x + v_off + h * vdim + 4 * g;
    float4 v = make_float4(to_f32(vx[0]), to_f32(vx[1]), to_f32(vx[2]), to_f32(vx[3]));
    if (FIXED) v = make_float4(silu_of(v.x), silu_of(v.y), silu_of(v.z), silu_of(v.w));
    __syncthreads();
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < ROWS; ++j) {
        if (j < rows_here) {
            const int i = row0 + j;
            const float a = as[i], k = ks[i], q = qs[i];
            s[j] = make_float4(a * s[j].x + k * v.x, a * s[j].y + k * v.y, a * s[j].z + k * v.z, a * s[j].w + k * v.w);
            o = make_float4(o.x + s[j].x * q, o.y + s[j].y * q, o.z + s[j].z * q, o.w + s[j].w * q);
            *reinterpret_cast<float4*>(S + (size_t)i * vdim) = s[j];
        }
    }
    if (r < slices) *reinterpret_cast<float4*>(red + r * vdim + 4 * g) = o;
    __syncthreads();
    float mine[2] = {0.f, 0.f};
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int c = tid + e * 256;
        if (c < vdim) {
            float t = 0.f;
            for (int rr = 0; rr < slices; ++rr) t += red[rr * vdim + c];
            mine[e] = t;
            ss += t * t;
            if (FIXED) raw[((size_t)b * heads + h) * vdim + c] = t;
        }
    }
    if (FIXED) return;
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)vdim + eps);
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int c = tid + e * 256;
        if (c < vdim) {
            const float gate = to_f32(x[g_off + h * vdim + c]);
            from_f32(out + ((size_t)b * heads + h) * vdim + c, mine[e] * inv * gain[c] * (gate / (1.0f + expf(-gate))));
        }
    }
}

// Whether the step kernel takes these head sizes: 1 yes, 0 no (then ri_gla_scan and ri_gla_norm_gate do).
extern "C" int ri_gla_step_fits(int dim, int vdim) {
    if (dim < 1 || dim > GLA_SLICES * GLA_MAX_ROWS || vdim < 4 || vdim % 4 || vdim > 512) return 0;
    const int groups = vdim / 4, slices = 256 / groups;
    return slices >= 1 && (dim + slices - 1) / slices <= GLA_STEP_ROWS && slices * vdim <= 1024;
}

extern "C" int ri_gla_step(void* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off, int g_off,
                           const float* z, const float* z_bias, float tau, float q_scale, float* state,
                           const int32_t* slots, const float* gain, float eps, int seqs, int heads, int dim, int vdim,
                           void* stream) {
    RI_REQUIRE(seqs > 0 && heads > 0 && ri_gla_step_fits(dim, vdim), "gla_step: %d sequences, %d heads of %d x %d", seqs,
               heads, dim, vdim);
    RI_REQUIRE(heads <= 65535 && seqs <= 65535, "gla_step: %d heads of %d sequences exceed one launch", heads, seqs);
    RI_REQUIRE(tau > 0.f, "gla_step: tau %g must be positive", (double)tau);
    RI_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && g_off >= 0 && q_off + heads * dim <= row && k_off + heads * dim <= row &&
               v_off + heads * vdim <= row && g_off + heads * vdim <= row,
               "gla_step: q, k, v, g at %d, %d, %d, %d do not fit rows of %d", q_off, k_off, v_off, g_off, row);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "gla_step: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    const int groups = vdim / 4, slices = 256 / groups;
    const dim3 grid(heads, seqs);
    const int rpt = (dim + slices - 1) / slices;
#define RI_STEP_GO(T, ROWS)                                                                                          \
    gla_step_kernel<T, ROWS, false><<<grid, 256, 0, s>>>((T*)out, (const T*)proj, row, q_off, k_off, v_off, g_off, z, z_bias, \
                                                  1.0f / tau, q_scale, state, slots, gain, eps, heads, dim, vdim, groups, \
                                                  slices, nullptr, nullptr)
    if (act_dtype == RI_F32) {
        if (rpt <= 8) RI_STEP_GO(float, 8); else if (rpt <= 16) RI_STEP_GO(float, 16); else RI_STEP_GO(float, 32);
    } else {
        if (rpt <= 8) RI_STEP_GO(bf16_t, 8); else if (rpt <= 16) RI_STEP_GO(bf16_t, 16); else RI_STEP_GO(bf16_t, 32);
    }
#undef RI_STEP_GO
    RI_LAUNCH_CHECK("gla_step");
    return 0;
}

// One new token a sequence of the linear attention with a fixed decay per head: the step on the state, the result as
// it is, float32 out[seqs][heads * vdim] (row b of proj belongs to slots[b]).  Head sizes as ri_gla_step_fits says.
extern "C" int ri_decay_step(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                             const float* head_decay, float q_scale, float* state, const int32_t* slots, int seqs,
                             int heads, int dim, int vdim, void* stream) {
    RI_REQUIRE(seqs > 0 && heads > 0 && ri_gla_step_fits(dim, vdim), "decay_step: %d sequences, %d heads of %d x %d", seqs,
               heads, dim, vdim);
    RI_REQUIRE(heads <= 65535 && seqs <= 65535, "decay_step: %d heads of %d sequences exceed one launch", heads, seqs);
    RI_REQUIRE(head_decay && out && state && slots, "decay_step: decays, a state and an output are needed");
    RI_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + heads * dim <= row && k_off + heads * dim <= row &&
               v_off + heads * vdim <= row, "decay_step: q, k, v at %d, %d, %d do not fit rows of %d", q_off, k_off, v_off, row);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "decay_step: dtype %d", act_dtype);
    hipStream_t s = (hipStream_t)stream;
    const int groups = vdim / 4, slices = 256 / groups;
    const dim3 grid(heads, seqs);
    const int rpt = (dim + slices - 1) / slices;
#define RI_STEP_GO(T, ROWS)                                                                                          \
    gla_step_kernel<T, ROWS, true><<<grid, 256, 0, s>>>(nullptr, (const T*)proj, row, q_off, k_off, v_off, 0, nullptr,   \
                                                 nullptr, 1.0f, q_scale, state, slots, nullptr, 0.f, heads, dim, vdim,   \
                                                 groups, slices, head_decay, out)
    if (act_dtype == RI_F32) {
        if (rpt <= 8) RI_STEP_GO(float, 8); else if (rpt <= 16) RI_STEP_GO(float, 16); else RI_STEP_GO(float, 32);
    } else {
        if (rpt <= 8) RI_STEP_GO(bf16_t, 8); else if (rpt <= 16) RI_STEP_GO(bf16_t, 16); else RI_STEP_GO(bf16_t, 32);
    }
#undef RI_STEP_GO
    RI_LAUNCH_CHECK("decay_step");
    return 0;
}
