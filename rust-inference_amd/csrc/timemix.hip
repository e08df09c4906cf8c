// Time mixing with a decay per key channel and a bonus for the current token, on a float32 state per sequence and head.
//
//   shift_mix:     with h' the row of the token before (the sequence's kept row for the first token of a step, zeros at a
//                  sequence's start), mix_s = h + (h' - h) * mu_s for every one of n mixing vectors mu_s: the inputs of
//                  the projections, one block of rows per s;
//   tanh_rows:     tanh of float32 rows, written in the activations' format (between the decay's two products);
//   shift_keep:    the last row of every sequence's step becomes its kept row (a launch of its own: the first token of a
//                  step reads the kept row while the last would write it);
//   timemix_scan:  per head, with r, k, v of a token and its decay w = exp(-exp(z + w0)) per key channel,
//                      o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,      S_t = diag(w_t) S_(t-1) + k_t v_t^T;
//                  then o is divided by its root mean square over the head, multiplied by the gain of its place among
//                  all heads and by silu(g), and written in the activations' format.
//
// The kept row, the mixes' arithmetic, the decay with both exponentials, the state, every sum of the recurrence and the
// norm are float32.  A workgroup owns one (sequence, head): a thread holds some rows of one column of the state in
// registers, the slices of rows meet through LDS in a fixed order, so a token's sums do not depend on how the tokens
// were cut into steps.  Any number of new tokens a sequence: the same kernel walks a prompt and takes a single step.
#include "api.h"
#include "common.h"

template <typename TA>
__global__ void __launch_bounds__(256)
shift_mix_kernel(TA* __restrict__ out, const float* __restrict__ x, const float* __restrict__ kept,
                 const float* __restrict__ mu, int n_mix, const int32_t* __restrict__ tok_seq,
                 const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots, int tokens, int width) {
    const int t = blockIdx.x;
    const int d = blockIdx.y * 256 + threadIdx.x;             // a thread an element: a single token is many short workgroups
    if (d >= width) return;
    const int seq = tok_seq[t];
    const float* before = t == cu_seqlens[seq] ? kept + (size_t)slots[seq] * width : x + (size_t)(t - 1) * width;
    const float h = x[(size_t)t * width + d], delta = before[d] - h;
    for (int s = 0; s < n_mix; ++s)
        from_f32(out + ((size_t)s * tokens + t) * width + d, h + delta * mu[(size_t)s * width + d]);
}

__global__ void __launch_bounds__(256)
shift_keep_kernel(float* __restrict__ kept, const float* __restrict__ x, const int32_t* __restrict__ cu_seqlens,
                  const int32_t* __restrict__ slots, int width) {
    const int seq = blockIdx.x;
    const int end = cu_seqlens[seq + 1];
    if (end == cu_seqlens[seq]) return;                       // a sequence without tokens keeps what it has
    for (int d = threadIdx.x; d < width; d += 256) kept[(size_t)slots[seq] * width + d] = x[(size_t)(end - 1) * width + d];
}

extern "C" int ri_shift_mix(void* out, int out_dtype, const float* x, const float* kept, const float* mu, int n_mix,
                            const int32_t* tok_seq, const int32_t* cu_seqlens, const int32_t* slots, int tokens, int width,
                            void* stream) {
    RI_REQUIRE(tokens > 0 && width > 0 && width <= 65535 * 256 && n_mix >= 1, "shift_mix: %d tokens of %d, %d mixes", tokens, width, n_mix);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "shift_mix: dtype %d", out_dtype);
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == RI_F32)
        shift_mix_kernel<float><<<dim3(tokens, (width + 255) / 256), 256, 0, s>>>((float*)out, x, kept, mu, n_mix, tok_seq, cu_seqlens, slots, tokens, width);
    else
        shift_mix_kernel<bf16_t><<<dim3(tokens, (width + 255) / 256), 256, 0, s>>>((bf16_t*)out, x, kept, mu, n_mix, tok_seq, cu_seqlens, slots, tokens, width);
    RI_LAUNCH_CHECK("shift_mix");
    return 0;
}

extern "C" int ri_shift_keep(float* kept, const float* x, const int32_t* cu_seqlens, const int32_t* slots, int seqs, int width,
                             void* stream) {
    RI_REQUIRE(seqs > 0 && width > 0, "shift_keep: %d sequences of %d", seqs, width);
    shift_keep_kernel<<<seqs, 256, 0, (hipStream_t)stream>>>(kept, x, cu_seqlens, slots, width);
    RI_LAUNCH_CHECK("shift_keep");
    return 0;
}

// out = tanh(x), float32 in, the activations' format out: between the two products of the decay's pre-activation.
template <typename TA>
__global__ void tanh_rows_kernel(TA* __restrict__ out, const float* __restrict__ x, long total) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < total) from_f32(out + e, tanhf(x[e]));
}

extern "C" int ri_tanh_rows(void* out, int out_dtype, const float* x, long total, void* stream) {
    RI_REQUIRE(total > 0 && (total + 255) / 256 <= 2147483647L, "tanh_rows: %ld elements", total);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "tanh_rows: dtype %d", out_dtype);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (out_dtype == RI_F32) tanh_rows_kernel<float><<<blocks, 256, 0, (hipStream_t)stream>>>((float*)out, x, total);
    else tanh_rows_kernel<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>((bf16_t*)out, x, total);
    RI_LAUNCH_CHECK("tanh_rows");
    return 0;
}

// ------------------------------------------------------------------ the walk
// blockDim.x = dim * slices; thread (slice, c) holds the rows slice * RPT .. + RPT - 1 of column c.
template <typename TA, int RPT>
__global__ void __launch_bounds__(1024)
timemix_scan_kernel(TA* __restrict__ out, int out_stride, int out_off, float out_scale, const TA* __restrict__ r,
                    const TA* __restrict__ k, const TA* __restrict__ v, const TA* __restrict__ g, const float* __restrict__ z,
                    const float* __restrict__ w0, const float* __restrict__ u, const float* __restrict__ gain, float eps,
                    float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots,
                    int heads, int dim, int slices) {
    extern __shared__ float lds[];
    float* rs = lds;                       // [dim] r
    float* ks = rs + dim;                  // [dim] k
    float* ws = ks + dim;                  // [dim] decay
    float* vs = ws + dim;                  // [dim] v
    float* red = vs + dim;                 // [slices][dim] the slices' shares of o
    float* os = red + (size_t)slices * dim;      // [dim] o
    const int seq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int c = tid % dim, slice = tid / dim;
    const int row0 = slice * RPT;
    const int width = heads * dim;
    float* sp = state + (((size_t)slots[seq] * heads + h) * dim) * dim;
    float st[RPT], ub[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int row = row0 + i;
        st[i] = row < dim ? sp[(size_t)row * dim + c] : 0.f;
        ub[i] = row < dim ? u[h * dim + row] : 0.f;
    }
    const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
    for (int t = t0; t < t1; ++t) {
        const size_t at = (size_t)t * width + (size_t)h * dim;
        __syncthreads();                                      // the token before has been read out of LDS
        if (tid < dim) {
            rs[tid] = to_f32(r[at + tid]);
            ks[tid] = to_f32(k[at + tid]);
            vs[tid] = to_f32(v[at + tid]);
            ws[tid] = expf(-expf(z[at + tid] + w0[h * dim + tid]));
        }
        __syncthreads();
        const float vc = vs[c];
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int row = row0 + i;
            if (row < dim) {
                const float kv = ks[row] * vc;
                part += (st[i] + ub[i] * kv) * rs[row];
                st[i] = ws[row] * st[i] + kv;
            }
        }
        red[slice * dim + c] = part;
        __syncthreads();
        if (tid < dim) {
            float o = 0.f;
            for (int s = 0; s < slices; ++s) o += red[s * dim + tid];
            os[tid] = o;
        }
        __syncthreads();
        if (tid < dim) {
            float ss = 0.f;
            for (int d = 0; d < dim; ++d) ss += os[d] * os[d];
            const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
            const float gate = to_f32(g[at + tid]);
            const float y = os[tid] * inv * gain[h * dim + tid] * (gate / (1.f + expf(-gate)));
            from_f32(out + (size_t)t * out_stride + out_off + (size_t)h * dim + tid, y * out_scale);
        }
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int row = row0 + i;
        if (row < dim) sp[(size_t)row * dim + c] = st[i];
    }
}

extern "C" int ri_timemix_max_dim() { return 256; }

extern "C" int ri_timemix_scan(void* out, int out_stride, int out_off, float out_scale, const void* r, const void* k,
                               const void* v, const void* g, int act_dtype, const float* z, const float* w0, const float* u,
                               const float* gain, float eps, float* state, const int32_t* cu_seqlens, const int32_t* slots,
                               int seqs, int heads, int dim, void* stream) {
    RI_REQUIRE(seqs > 0 && heads > 0 && heads <= 65535 && dim >= 1 && dim <= 256, "timemix_scan: %d sequences, %d heads of %d", seqs,
               heads, dim);
    RI_REQUIRE(out_off >= 0 && out_off + heads * dim <= out_stride, "timemix_scan: column %d of rows of %d", out_off, out_stride);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "timemix_scan: dtype %d", act_dtype);
    // slices of rows: as many as keep a thread's rows at 32 or fewer, within 1,024 threads
    int slices = (dim + 31) / 32;
    while (slices * 2 * dim <= 256) slices *= 2;             // small heads: fill four wavefronts
    if (slices > dim) slices = dim;
    while (slices > 1 && slices * dim > 1024) slices /= 2;
    const int rpt = (dim + slices - 1) / slices;
    RI_REQUIRE(slices * dim <= 1024 && rpt <= 64, "timemix_scan: heads of %d do not fit a workgroup", dim);
    const dim3 grid(seqs, heads);
    const int threads = slices * dim;
    const size_t lds = ((size_t)5 * dim + (size_t)slices * dim) * sizeof(float);
    hipStream_t s = (hipStream_t)stream;
#define RI_GO(TA, RPT)                                                                                                  \
    timemix_scan_kernel<TA, RPT><<<grid, threads, lds, s>>>((TA*)out, out_stride, out_off, out_scale, (const TA*)r,     \
                                                            (const TA*)k, (const TA*)v, (const TA*)g, z, w0, u, gain, eps, \
                                                            state, cu_seqlens, slots, heads, dim, slices)
#define RI_BY_ROWS(TA)                                                                                                  \
    if (rpt <= 8) RI_GO(TA, 8); else if (rpt <= 16) RI_GO(TA, 16); else if (rpt <= 32) RI_GO(TA, 32); else RI_GO(TA, 64)
    if (act_dtype == RI_F32) { RI_BY_ROWS(float); } else { RI_BY_ROWS(bf16_t); }
#undef RI_BY_ROWS
#undef RI_GO
    RI_LAUNCH_CHECK("timemix_scan");
    return 0;
}

// ------------------------------------------------------------------ the walk, a wavefront on 16 columns
// Heads of up to 128: a wavefront owns 16 columns of one (sequence, head), its lanes four slices of the rows of a column
// each (8 columns and eight slices for heads above 64: a token's walk over a lane's rows is what the wavefront waits for), the rows in registers; a token's sum over the rows is the lane's own sum (four partial sums, so that no addition
// waits for the one before) and two exchanges between the lanes of a column.  A workgroup is four wavefronts on columns of
// their own, which share the tokens staged in LDS in blocks of TM_BLOCK (r, k, the decay, v), the next block's loads asked for before the block in work is
// computed.  The heads' results are written as they are, float32; the norm over a head and the gate are
// heads_norm_gate's.
#define TM_BLOCK 8
#define TM_WAVES 4           // wavefronts of a workgroup: they share the staged tokens, each on columns of its own

template <typename TA, int RPL, int SL>                       // RPL: rows a lane holds, a multiple of 4; SL: slices of rows, 4 or 8
__global__ void __launch_bounds__(64 * TM_WAVES)
timemix_scan_cols_kernel(float* __restrict__ out, const TA* __restrict__ r, const TA* __restrict__ k, const TA* __restrict__ v,
                         const float* __restrict__ z, const float* __restrict__ u,
                         float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots,
                         int heads, int dim) {
    // COLS: columns of a wavefront; NC: of the workgroup; TPP: tokens whose v one pass of the workgroup's threads fetches
    constexpr int ROWS = SL * RPL, COLS = 64 / SL, NC = COLS * TM_WAVES, THREADS = 64 * TM_WAVES, TPP = THREADS / NC,
                  PASSES = TM_BLOCK / TPP;
    __shared__ __attribute__((aligned(16))) float rs[2][TM_BLOCK][ROWS];
    __shared__ __attribute__((aligned(16))) float ks[2][TM_BLOCK][ROWS];
    __shared__ __attribute__((aligned(16))) float ws[2][TM_BLOCK][ROWS];
    __shared__ float vs[2][TM_BLOCK][NC];
    const int seq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane % COLS, slice = lane / COLS, row0 = slice * RPL;
    const int wcol = wave * COLS + col;                       // the lane's column among the workgroup's
    const int c = blockIdx.z * NC + wcol;
    const bool has_col = c < dim;
    const int cc = has_col ? c : dim - 1;                     // a column pulled back inside the head: loads are issued anyway
    const int width = heads * dim;
    float* sp = state + (((size_t)slots[seq] * heads + h) * dim) * dim + cc;
    float st[RPL], ub[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        st[i] = row0 + i < dim ? sp[(size_t)(row0 + i) * dim] : 0.f;
        ub[i] = row0 + i < dim ? u[h * dim + row0 + i] : 0.f;
    }
    const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
    constexpr int PER = (TM_BLOCK * ROWS + THREADS - 1) / THREADS;      // elements of each of r, k and the decay that a thread stages
    const int vcol = min((int)blockIdx.z * NC + tid % NC, dim - 1), vtok = tid / NC;      // the thread's place in a pass over v

    float pre_r[PER], pre_k[PER], pre_w[PER], pre_v[PASSES];
    auto fetch = [&](int tb) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = tid + i * THREADS;
            const int row = e % ROWS, tt = e / ROWS;
            const bool in = row < dim && tt < TM_BLOCK;
            const size_t at = (size_t)min(tb + tt, t1 - 1) * width + (size_t)h * dim + (in ? row : 0);
            pre_r[i] = in ? to_f32(r[at]) : 0.f;
            pre_k[i] = in ? to_f32(k[at]) : 0.f;
            pre_w[i] = in ? z[at] : 0.f;                     // the decay itself: timemix_decay has been over z
        }
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps)
            pre_v[ps] = to_f32(v[(size_t)min(tb + ps * TPP + vtok, t1 - 1) * width + (size_t)h * dim + vcol]);
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = tid + i * THREADS;
            const int row = e % ROWS, tt = e / ROWS;
            if (tt < TM_BLOCK) {
                rs[buf][tt][row] = pre_r[i];
                ks[buf][tt][row] = pre_k[i];
                ws[buf][tt][row] = pre_w[i];
            }
        }
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) vs[buf][ps * TPP + vtok][tid % NC] = pre_v[ps];
    };
    if (t0 < t1) {
        fetch(t0);
        stage(0);
    }
    __syncthreads();
    int buf = 0;
    for (int tb = t0; tb < t1; tb += TM_BLOCK, buf ^= 1) {
        const bool more = tb + TM_BLOCK < t1;
        if (more) fetch(tb + TM_BLOCK);
        const int count = min(TM_BLOCK, t1 - tb);
        float part[TM_BLOCK];                                 // the lane's share of each token's sum: the exchanges wait for the block's end,
#pragma unroll                                                // so that no token waits for the one before it
        for (int tt = 0; tt < TM_BLOCK; ++tt) {
            part[tt] = 0.f;
            if (tt < count) {
                const float vc = vs[buf][tt][wcol];
                float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
                for (int i = 0; i < RPL; i += 4) {
                    const float4 r4 = *reinterpret_cast<const float4*>(&rs[buf][tt][row0 + i]);
                    const float4 k4 = *reinterpret_cast<const float4*>(&ks[buf][tt][row0 + i]);
                    const float4 w4 = *reinterpret_cast<const float4*>(&ws[buf][tt][row0 + i]);
                    float kv = k4.x * vc;
                    o0 += (st[i] + ub[i] * kv) * r4.x;               st[i] = w4.x * st[i] + kv;
                    kv = k4.y * vc;
                    o1 += (st[i + 1] + ub[i + 1] * kv) * r4.y;       st[i + 1] = w4.y * st[i + 1] + kv;
                    kv = k4.z * vc;
                    o2 += (st[i + 2] + ub[i + 2] * kv) * r4.z;       st[i + 2] = w4.z * st[i + 2] + kv;
                    kv = k4.w * vc;
                    o3 += (st[i + 3] + ub[i + 3] * kv) * r4.w;       st[i + 3] = w4.w * st[i + 3] + kv;
                }
                part[tt] = (o0 + o1) + (o2 + o3);
            }
        }
#pragma unroll
        for (int tt = 0; tt < TM_BLOCK; ++tt) {
            float o = part[tt];
            if (SL == 8) o += __shfl_xor(o, 8, RI_WAVE);      // the slices of a column
            o += __shfl_xor(o, 16, RI_WAVE);
            o += __shfl_xor(o, 32, RI_WAVE);
            if (tt < count && has_col && slice == 0) out[(size_t)(tb + tt) * width + (size_t)h * dim + c] = o;
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    }
    if (has_col) {
#pragma unroll
        for (int i = 0; i < RPL; ++i)
            if (row0 + i < dim) sp[(size_t)(row0 + i) * dim] = st[i];
    }
}

// out[t, out_off + h * dim + c] = scale * o[t, h, c] / sqrt(mean_c(o[t, h, :]^2) + eps) * gain[h * dim + c] * silu(g[t, h * dim + c]).
template <typename TA>
__global__ void __launch_bounds__(64)
heads_norm_gate_kernel(TA* __restrict__ out, int out_stride, int out_off, float scale, const float* __restrict__ o,
                       const float* __restrict__ gain, const TA* __restrict__ g, float eps, int heads, int dim) {
    const int t = blockIdx.x, h = blockIdx.y;
    const size_t at = ((size_t)t * heads + h) * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 64) ss += o[at + d] * o[at + d];
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += 64) {
        const float gate = to_f32(g[at + d]);
        from_f32(out + (size_t)t * out_stride + out_off + (size_t)h * dim + d,
                 o[at + d] * inv * gain[h * dim + d] * (gate / (1.f + expf(-gate))) * scale);
    }
}

// z <- exp(-exp(z + w0)) in place: every token's decays once, before the walk, whose sixteen wavefronts a head would each
// take both exponentials again.
__global__ void timemix_decay_kernel(float* __restrict__ z, const float* __restrict__ w0, long total, int width) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < total) z[e] = expf(-expf(z[e] + w0[e % width]));
}

extern "C" int ri_timemix_scan_cols_fits(int dim) { return dim >= 1 && dim <= 128; }

extern "C" int ri_timemix_scan_cols(void* out, int out_stride, int out_off, float out_scale, float* o, const void* r,
                                    const void* k, const void* v, const void* g, int act_dtype, float* z, const float* w0,
                                    const float* u, const float* gain, float eps, float* state, const int32_t* cu_seqlens,
                                    const int32_t* slots, int tokens, int seqs, int heads, int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && seqs > 0 && heads > 0 && heads <= 65535 && ri_timemix_scan_cols_fits(dim),
               "timemix_scan_cols: %d tokens of %d sequences, %d heads of %d", tokens, seqs, heads, dim);
    RI_REQUIRE(out_off >= 0 && out_off + heads * dim <= out_stride, "timemix_scan_cols: column %d of rows of %d", out_off, out_stride);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "timemix_scan_cols: dtype %d", act_dtype);
    const int cols = (dim > 64 ? 8 : 16) * TM_WAVES;
    const dim3 grid(seqs, heads, (dim + cols - 1) / cols);
    hipStream_t s = (hipStream_t)stream;
    const long total = (long)tokens * heads * dim;
    RI_REQUIRE((total + 255) / 256 <= 2147483647L, "timemix_scan_cols: %ld decays exceed one launch", total);
    timemix_decay_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(z, w0, total, heads * dim);
#define RI_GO(TA, ROWS, SL)                                                                                             \
    timemix_scan_cols_kernel<TA, ROWS, SL><<<grid, 64 * TM_WAVES, 0, s>>>(o, (const TA*)r, (const TA*)k, (const TA*)v, z, u, state,  \
                                                           cu_seqlens, slots, heads, dim)
#define RI_BY_ROWS(TA)                                                                                                  \
    if (dim <= 16) RI_GO(TA, 4, 4); else if (dim <= 32) RI_GO(TA, 8, 4); else if (dim <= 64) RI_GO(TA, 16, 4); else RI_GO(TA, 16, 8)
    if (act_dtype == RI_F32) {
        RI_BY_ROWS(float);
        heads_norm_gate_kernel<float><<<dim3(tokens, heads), 64, 0, s>>>((float*)out, out_stride, out_off, out_scale, o, gain,
                                                                        (const float*)g, eps, heads, dim);
    } else {
        RI_BY_ROWS(bf16_t);
        heads_norm_gate_kernel<bf16_t><<<dim3(tokens, heads), 64, 0, s>>>((bf16_t*)out, out_stride, out_off, out_scale, o, gain,
                                                                         (const bf16_t*)g, eps, heads, dim);
    }
#undef RI_BY_ROWS
#undef RI_GO
    RI_LAUNCH_CHECK("timemix_scan_cols");
    return 0;
}
