// Linear attention with one fixed decay per head over prompts, in chunks of 64 tokens instead of token by token:
//     S_t = d S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   q = silu(.) * q_scale, k = silu(.), v = silu(.).
// With a decay that is a constant the tokens of a chunk need not wait for one another.  For a chunk of n tokens that
// starts from the state S0,
//     o_i   = sum_{j <= i} d^(i - j) (q_i . k_j) v_j  +  d^(i + 1) S0^T q_i,
//     S_end = d^n S0 + sum_j d^(n - 1 - j) k_j v_j^T,
// so a step is three launches: every chunk's own sum U = sum_j d^(n - 1 - j) k_j v_j^T (all chunks side by side), the
// walk from chunk to chunk, S0 of the next = d^n S0 + U, which leaves every chunk's S0 where its U was and the last
// state in the sequence's slot (a few loads and stores an element), and every chunk's outputs (all chunks side by side).
// Only powers d^m with m >= 0 appear, so no decay is too small or too large for it.  Everything is float32: the
// activations after silu, the powers, the scores q . k, the state and all sums; a sum runs over its tokens or channels
// in their order.  A workgroup of 512 threads takes one (chunk, sequence, head); a thread keeps tiles of 4 x 4 results
// and reads its operands from LDS 16 bytes at a time.  Head sizes: multiples of 4 up to 128.
#include "api.h"
#include "common.h"

#define DC_TOK 64                // tokens of a chunk
#define DC_MAX 128               // largest key or value head
#define DC_SLAB 32               // rows of S0 staged at a time
#define DC_ASTRIDE (DC_TOK + 4)
#define DC_THREADS 512           // of the workgroups that work on a chunk: two wavefronts a SIMD, one behind the other's loads
#define DC_STAGED (DC_TOK * DC_MAX / 4 / DC_THREADS)    // most 16-byte pieces a thread stages of one operand

__device__ __forceinline__ float dc_silu(float v) { return v / (1.0f + expf(-v)); }

__device__ __forceinline__ float4 dc_ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 dc_ld4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16),
                       __uint_as_float(w.y & 0xFFFF0000u));
}

// The workspace's entry of chunk c of sequence b, which starts at token t0 of the step: sequences' entries do not
// meet, since a sequence of len tokens has at most len / 64 + 1 chunks.
__device__ __forceinline__ size_t dc_entry(int t0, int b, int c) { return (size_t)(t0 / DC_TOK + b + c); }

// Rows of `width` activations of tokens first .. first + n - 1 (columns col0 .. of proj's rows) through silu into LDS
// rows of `stride` floats, times factor * d^(n - 1 - j) with pw (pw == nullptr: times factor alone); rows n .. 63 zero.
// Loads are issued whatever the indices are, from a token pulled back inside the chunk.
template <typename TA>
__device__ __forceinline__ void dc_stage(float* dst, int stride, const TA* __restrict__ proj, int row, int col0, int first,
                                         int n, int width, float factor, const float* pw) {
    const int per = width / 4, total = DC_TOK * per;
    float4 x[DC_STAGED];
    int tok[DC_STAGED], at[DC_STAGED];
    // all of a thread's loads are asked for before the first is used
#pragma unroll
    for (int it = 0; it < DC_STAGED; ++it) {
        const int e = min((int)threadIdx.x + it * DC_THREADS, total - 1);
        tok[it] = e / per;
        at[it] = (e - tok[it] * per) * 4;
        x[it] = dc_ld4(proj + (size_t)(first + min(tok[it], n - 1)) * row + col0 + at[it]);
    }
#pragma unroll
    for (int it = 0; it < DC_STAGED; ++it) {
        if ((int)threadIdx.x + it * DC_THREADS < total) {
            const int j = tok[it];
            const float f = j < n ? factor * (pw ? pw[n - 1 - j] : 1.0f) : 0.f;
            float4 y;
            y.x = j < n ? dc_silu(x[it].x) * f : 0.f;
            y.y = j < n ? dc_silu(x[it].y) * f : 0.f;
            y.z = j < n ? dc_silu(x[it].z) * f : 0.f;
            y.w = j < n ? dc_silu(x[it].w) * f : 0.f;
            *reinterpret_cast<float4*>(dst + j * stride + at[it]) = y;
        }
    }
}

// pw[m] = d^m for m = 0 .. 64 (d^0 = 1 also for d = 0).
__device__ __forceinline__ void dc_powers(float* pw, float d) {
    if (threadIdx.x <= DC_TOK) pw[threadIdx.x] = threadIdx.x == 0 ? 1.0f : powf(d, (float)threadIdx.x);
}

// U[entry, h] = sum_j d^(n - 1 - j) k_j v_j^T   [dim, vdim]
template <typename TA>
__global__ void __launch_bounds__(DC_THREADS)
decay_chunk_sums_kernel(float* __restrict__ U, const TA* __restrict__ proj, int row, int k_off, int v_off,
                        const int32_t* __restrict__ cu_seqlens, const float* __restrict__ head_decay, int heads, int dim,
                        int vdim) {
    extern __shared__ __align__(16) float lds[];           // read 16 bytes at a time: it must start on a multiple of 16,
    __shared__ __align__(16) float pw[DC_TOK + 4];         // so what stands before it is a multiple of 16 bytes too
    const int c = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
    const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
    const int first = t0 + c * DC_TOK;
    if (first >= t1) return;
    const int n = min(DC_TOK, t1 - first);
    float* Ks = lds;                       // [64][dim], already times d^(n - 1 - j)
    float* Vs = lds + DC_TOK * dim;        // [64][vdim]
    dc_powers(pw, head_decay[h]);
    __syncthreads();
    dc_stage(Ks, dim, proj, row, k_off + h * dim, first, n, dim, 1.0f, pw);
    dc_stage(Vs, vdim, proj, row, v_off + h * vdim, first, n, vdim, 1.0f, (const float*)nullptr);
    __syncthreads();
    float* Uc = U + (dc_entry(t0, b, c) * heads + h) * dim * vdim;
    const int tcs = vdim / 4, tiles = (dim / 4) * tcs;
    for (int tile = threadIdx.x; tile < tiles; tile += DC_THREADS) {
        const int tr = tile / tcs, tc = tile - tr * tcs;
        float acc[4][4] = {};
        for (int j0 = 0; j0 < n; j0 += 4) {                  // (the rows from n on are zeros)
            float4 k4[4], v4[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                k4[m] = *reinterpret_cast<const float4*>(Ks + (j0 + m) * dim + 4 * tr);
                v4[m] = *reinterpret_cast<const float4*>(Vs + (j0 + m) * vdim + 4 * tc);
            }
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float kk[4] = {k4[m].x, k4[m].y, k4[m].z, k4[m].w};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    acc[r][0] += kk[r] * v4[m].x;
                    acc[r][1] += kk[r] * v4[m].y;
                    acc[r][2] += kk[r] * v4[m].z;
                    acc[r][3] += kk[r] * v4[m].w;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
            *reinterpret_cast<float4*>(Uc + (size_t)(4 * tr + r) * vdim + 4 * tc) = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
    }
}

// From chunk to chunk: every chunk's entry gets the state it starts from, the slot the state after the last token.
__global__ void __launch_bounds__(256)
decay_chunk_carry_kernel(float* __restrict__ U, float* __restrict__ state, const int32_t* __restrict__ cu_seqlens,
                         const int32_t* __restrict__ slots, const float* __restrict__ head_decay, int heads, int dim,
                         int vdim) {
    const int b = blockIdx.y, h = blockIdx.z;
    const int e = (blockIdx.x * 256 + threadIdx.x) * 4, size = dim * vdim;
    const int t0 = cu_seqlens[b], len = cu_seqlens[b + 1] - t0;
    if (e >= size || len <= 0) return;
    const float d = head_decay[h], whole = powf(d, (float)DC_TOK);
    float* Sp = state + ((size_t)slots[b] * heads + h) * size + e;
    float4 s = *reinterpret_cast<const float4*>(Sp);
    const int chunks = (len + DC_TOK - 1) / DC_TOK;
    float* Up = U + (dc_entry(t0, b, 0) * heads + h) * size + e;
    const size_t step = (size_t)heads * size;
    float4 u = *reinterpret_cast<const float4*>(Up);
    for (int c = 0; c < chunks; ++c) {
        // the next chunk's sum is asked for before this one's place is written (the last chunk asks for its own again)
        const float4 next = *reinterpret_cast<const float4*>(Up + (size_t)min(c + 1, chunks - 1) * step);
        *reinterpret_cast<float4*>(Up + (size_t)c * step) = s;
        const int n = min(DC_TOK, len - c * DC_TOK);
        const float f = n == DC_TOK ? whole : powf(d, (float)n);
        s.x = f * s.x + u.x;
        s.y = f * s.y + u.y;
        s.z = f * s.z + u.z;
        s.w = f * s.w + u.w;
        u = next;
    }
    *reinterpret_cast<float4*>(Sp) = s;
}

// o_i = sum_{j <= i} d^(i - j) (q_i . k_j) v_j + d^(i + 1) S0^T q_i for the tokens of one chunk.
template <typename TA>
__global__ void __launch_bounds__(DC_THREADS)
decay_chunk_out_kernel(float* __restrict__ out, const float* __restrict__ U, const TA* __restrict__ proj, int row, int q_off,
                       int k_off, int v_off, const int32_t* __restrict__ cu_seqlens, const float* __restrict__ head_decay,
                       float q_scale, int heads, int dim, int vdim) {
    extern __shared__ __align__(16) float lds[];           // read 16 bytes at a time: it must start on a multiple of 16,
    __shared__ __align__(16) float pw[DC_TOK + 4];         // so what stands before it is a multiple of 16 bytes too
    const int c = blockIdx.x, b = blockIdx.y, h = blockIdx.z, tid = threadIdx.x;
    const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
    const int first = t0 + c * DC_TOK;
    if (first >= t1) return;
    const int n = min(DC_TOK, t1 - first);
    const int qs = dim + 4;                                  // row stride of Q and K
    float* Qs = lds;                                         // [64][dim + 4]
    float* KV = Qs + DC_TOK * qs;                            // K [64][dim + 4], later V [64][vdim]
    float* As = KV + DC_TOK * max(qs, vdim);                 // [64][68]: the scores times the decay's powers
    float* Ss = As + DC_TOK * DC_ASTRIDE;                    // [32][vdim]: a slab of S0's rows
    dc_powers(pw, head_decay[h]);
    dc_stage(Qs, qs, proj, row, q_off + h * dim, first, n, dim, q_scale, (const float*)nullptr);
    dc_stage(KV, qs, proj, row, k_off + h * dim, first, n, dim, 1.0f, (const float*)nullptr);
    __syncthreads();
    {   // scores: thread (ti, tj) takes queries 4 ti .. 4 ti + 3 and keys tj and tj + 32
        const int ti = tid / 32, tj = tid % 32;
        float acc[4][2] = {};
        for (int k = 0; k < dim; k += 4) {
            float4 q4[4], k4[2];
#pragma unroll
            for (int r = 0; r < 4; ++r) q4[r] = *reinterpret_cast<const float4*>(Qs + (4 * ti + r) * qs + k);
#pragma unroll
            for (int s = 0; s < 2; ++s) k4[s] = *reinterpret_cast<const float4*>(KV + (tj + 32 * s) * qs + k);
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    acc[r][s] += q4[r].x * k4[s].x + q4[r].y * k4[s].y + q4[r].z * k4[s].z + q4[r].w * k4[s].w;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int i = 4 * ti + r, j = tj + 32 * s;
                As[i * DC_ASTRIDE + j] = (j <= i && i < n) ? acc[r][s] * pw[i - min(j, i)] : 0.f;
            }
    }
    __syncthreads();                                         // the keys have been read: the values take their place
    dc_stage(KV, vdim, proj, row, v_off + h * vdim, first, n, vdim, 1.0f, (const float*)nullptr);
    __syncthreads();
    // results: tiles of 4 tokens x 4 columns, at most one a thread
    const int tcs = vdim / 4, tiles = (DC_TOK / 4) * tcs;
    float acc[1][4][4] = {}, from_state[1][4][4] = {};
#pragma unroll
    for (int w = 0; w < 1; ++w) {
        const int tile = tid + w * DC_THREADS;
        if (tile < tiles) {
            const int ti = tile / tcs, tc = tile - ti * tcs;
            for (int j = 0; j < DC_TOK; j += 4) {
                float4 a4[4], v4[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    a4[r] = *reinterpret_cast<const float4*>(As + (4 * ti + r) * DC_ASTRIDE + j);
                    v4[r] = *reinterpret_cast<const float4*>(KV + (j + r) * vdim + 4 * tc);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float a[4] = {a4[r].x, a4[r].y, a4[r].z, a4[r].w};
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        acc[w][r][0] += a[m] * v4[m].x;
                        acc[w][r][1] += a[m] * v4[m].y;
                        acc[w][r][2] += a[m] * v4[m].z;
                        acc[w][r][3] += a[m] * v4[m].w;
                    }
                }
            }
        }
    }
    const float* S0 = U + (dc_entry(t0, b, c) * heads + h) * dim * vdim;
    for (int k0 = 0; k0 < dim; k0 += DC_SLAB) {
        const int rows = min(DC_SLAB, dim - k0);             // a multiple of 4
        __syncthreads();                                     // the slab before has been read
        for (int e = tid; e < rows * tcs; e += DC_THREADS)
            *reinterpret_cast<float4*>(Ss + e * 4) = *reinterpret_cast<const float4*>(S0 + (size_t)k0 * vdim + e * 4);
        __syncthreads();
#pragma unroll
        for (int w = 0; w < 1; ++w) {
            const int tile = tid + w * DC_THREADS;
            if (tile < tiles) {
                const int ti = tile / tcs, tc = tile - ti * tcs;
                for (int k = 0; k < rows; k += 4) {
                    float4 q4[4], s4[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        q4[r] = *reinterpret_cast<const float4*>(Qs + (4 * ti + r) * qs + k0 + k);
                        s4[r] = *reinterpret_cast<const float4*>(Ss + (k + r) * vdim + 4 * tc);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float q[4] = {q4[r].x, q4[r].y, q4[r].z, q4[r].w};
#pragma unroll
                        for (int m = 0; m < 4; ++m) {
                            from_state[w][r][0] += q[m] * s4[m].x;
                            from_state[w][r][1] += q[m] * s4[m].y;
                            from_state[w][r][2] += q[m] * s4[m].z;
                            from_state[w][r][3] += q[m] * s4[m].w;
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int w = 0; w < 1; ++w) {
        const int tile = tid + w * DC_THREADS;
        if (tile < tiles) {
            const int ti = tile / tcs, tc = tile - ti * tcs;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * ti + r;
                if (i < n) {
                    const float f = pw[i + 1];
                    *reinterpret_cast<float4*>(out + (size_t)(first + i) * heads * vdim + h * vdim + 4 * tc) =
                        make_float4(acc[w][r][0] + f * from_state[w][r][0], acc[w][r][1] + f * from_state[w][r][1],
                                    acc[w][r][2] + f * from_state[w][r][2], acc[w][r][3] + f * from_state[w][r][3]);
                }
            }
        }
    }
}

extern "C" int ri_decay_chunks_fit(int dim, int vdim) {
    return dim >= 4 && vdim >= 4 && dim <= DC_MAX && vdim <= DC_MAX && dim % 4 == 0 && vdim % 4 == 0;
}

// How many floats of workspace a step of `tokens` tokens in `seqs` sequences needs.
extern "C" long ri_decay_chunks_workspace(int seqs, int tokens, int heads, int dim, int vdim) {
    return ((long)tokens / DC_TOK + seqs) * heads * dim * vdim;
}

extern "C" int ri_decay_scan_chunked(float* out, const void* proj, int act_dtype, int row, int q_off, int k_off, int v_off,
                                     const float* head_decay, float q_scale, float* state, const int32_t* cu_seqlens,
                                     const int32_t* slots, int seqs, int tokens, int max_new, int heads, int dim, int vdim,
                                     float* workspace, long workspace_floats, void* stream) {
    RI_REQUIRE(out && proj && head_decay && state && cu_seqlens && slots && workspace, "decay_scan_chunked: a null pointer");
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "decay_scan_chunked: dtype %d", act_dtype);
    RI_REQUIRE(ri_decay_chunks_fit(dim, vdim), "decay_scan_chunked: heads of %d x %d (multiples of 4 up to %d)", dim, vdim, DC_MAX);
    RI_REQUIRE(seqs >= 1 && tokens >= seqs && heads >= 1 && heads <= 65535 && seqs <= 65535 && max_new >= 1 && max_new <= tokens,
               "decay_scan_chunked: %d tokens in %d sequences of at most %d, %d heads", tokens, seqs, max_new, heads);
    RI_REQUIRE(row % 4 == 0 && q_off % 4 == 0 && k_off % 4 == 0 && v_off % 4 == 0 && q_off >= 0 && k_off >= 0 && v_off >= 0 &&
               q_off + heads * dim <= row && k_off + heads * dim <= row && v_off + heads * vdim <= row,
               "decay_scan_chunked: columns %d, %d, %d of rows of %d (multiples of 4)", q_off, k_off, v_off, row);
    RI_REQUIRE(workspace_floats >= ri_decay_chunks_workspace(seqs, tokens, heads, dim, vdim),
               "decay_scan_chunked: a workspace of %ld floats", workspace_floats);
    hipStream_t s = (hipStream_t)stream;
    const int chunks = (max_new + DC_TOK - 1) / DC_TOK;
    const dim3 grid(chunks, seqs, heads);
    const size_t lds_sums = (size_t)DC_TOK * (dim + vdim) * sizeof(float);
    const size_t lds_out = ((size_t)DC_TOK * (dim + 4) + (size_t)DC_TOK * (dim + 4 > vdim ? dim + 4 : vdim) +
                            (size_t)DC_TOK * DC_ASTRIDE + (size_t)DC_SLAB * vdim) * sizeof(float);
#define RI_DC_GO(T)                                                                                                  \
    {                                                                                                                \
        static bool asked = false;                                                                                   \
        if (!asked) {                                                                                                \
            hipError_t e_ = hipFuncSetAttribute((const void*)decay_chunk_sums_kernel<T>,                             \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);             \
            RI_REQUIRE(e_ == hipSuccess, "decay_scan_chunked: %s", hipGetErrorString(e_));                           \
            e_ = hipFuncSetAttribute((const void*)decay_chunk_out_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                     128 * 1024);                                                                    \
            RI_REQUIRE(e_ == hipSuccess, "decay_scan_chunked: %s", hipGetErrorString(e_));                           \
            asked = true;                                                                                            \
        }                                                                                                            \
        decay_chunk_sums_kernel<T><<<grid, DC_THREADS, lds_sums, s>>>(workspace, (const T*)proj, row, k_off, v_off, cu_seqlens, \
                                                               head_decay, heads, dim, vdim);                        \
        decay_chunk_carry_kernel<<<dim3((dim * vdim / 4 + 255) / 256, seqs, heads), 256, 0, s>>>(                    \
            workspace, state, cu_seqlens, slots, head_decay, heads, dim, vdim);                                      \
        decay_chunk_out_kernel<T><<<grid, DC_THREADS, lds_out, s>>>(out, workspace, (const T*)proj, row, q_off, k_off, v_off, \
                                                             cu_seqlens, head_decay, q_scale, heads, dim, vdim);     \
    }
    if (act_dtype == RI_F32) RI_DC_GO(float) else RI_DC_GO(bf16_t)
#undef RI_DC_GO
    RI_LAUNCH_CHECK("decay_scan_chunked");
    return 0;
}
