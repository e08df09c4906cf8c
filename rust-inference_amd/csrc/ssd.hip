// A state-space mixer with a scalar decay per head (the structured state-space duality form), on a float32 state per
// sequence and head.
//
//   causal_conv_silu:  every channel's causal convolution over the tokens of its sequence, bias, silu; the inputs before
//                      a step's first token come from the sequence's kept tail (its last taps - 1 inputs, oldest first,
//                      zeros at a sequence's start); the taps are added oldest first, the current token's last;
//   conv_tails:        moves every sequence's tail on by the step's tokens (a launch of its own: the first tokens of a
//                      step read the tail that the last ones would write);
//   ssd_scan:          per head h (which reads B and C of group h / (heads / groups)), with dt = softplus(dt_raw + dt_bias_h):
//                          S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T,      y_t = S_t^T C_t + D_h x_t,
//                      then y times silu(z), float32;
//   group_rms_norm:    a row in equal parts, each divided by its own root mean square, times a gain an element.
//
// The step size with its softplus, the decay with both exponentials, the state, every sum of the recurrence, the gate and
// the norm are float32.  A workgroup of ssd_scan owns one (sequence, head): a thread holds some rows of one column of
// the state in registers and the slices of rows meet through LDS in a fixed order, so a token's sums do not depend on
// how the tokens were cut into steps.  The same kernels walk a prompt and take a single step.
#include "api.h"
#include "common.h"

#define SSD_MAX_TAPS 16

template <typename TA>
__global__ void __launch_bounds__(256)
causal_conv_silu_kernel(float* __restrict__ out, const TA* __restrict__ proj, int stride, int col0, const float* __restrict__ taps_w,
                        const float* __restrict__ bias, const float* __restrict__ tails, int taps,
                        const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ cu_seqlens,
                        const int32_t* __restrict__ slots, int channels) {
    const int t = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
    if (ch >= channels) return;
    const int seq = tok_seq[t];
    const int first = cu_seqlens[seq];
    const int i = t - first;                                  // the token's place in this step
    const float* tail = tails + (size_t)slots[seq] * (taps - 1) * channels;
    float sum = 0.f;
    for (int a = 0; a < taps; ++a) {                          // oldest first
        const int src = i - (taps - 1 - a);
        const float in = src >= 0 ? to_f32(proj[(size_t)(first + src) * stride + col0 + ch])
                                  : tail[(size_t)(taps - 1 + src) * channels + ch];
        sum += in * taps_w[(size_t)ch * taps + a];
    }
    if (bias) sum += bias[ch];
    out[(size_t)t * channels + ch] = sum / (1.f + expf(-sum));
}

template <typename TA>
__global__ void __launch_bounds__(256)
conv_tails_kernel(float* __restrict__ tails, const TA* __restrict__ proj, int stride, int col0, int taps,
                  const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots, int channels) {
    const int seq = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
    if (ch >= channels) return;
    const int first = cu_seqlens[seq], n = cu_seqlens[seq + 1] - first;
    if (n == 0) return;
    float* tail = tails + (size_t)slots[seq] * (taps - 1) * channels;
    float keep[SSD_MAX_TAPS];
    for (int idx = 0; idx < taps - 1; ++idx) {
        const int src = n - (taps - 1) + idx;                 // the step's token that lands at this place, if any
        keep[idx] = src >= 0 ? to_f32(proj[(size_t)(first + src) * stride + col0 + ch])
                             : tail[(size_t)(idx + n) * channels + ch];
    }
    for (int idx = 0; idx < taps - 1; ++idx) tail[(size_t)idx * channels + ch] = keep[idx];
}

extern "C" int ri_causal_conv_silu(float* out, const void* proj, int act_dtype, int stride, int col0, const float* taps_w,
                                   const float* bias, float* tails, int taps, const int32_t* tok_seq, const int32_t* cu_seqlens,
                                   const int32_t* slots, int tokens, int seqs, int channels, int update_tails, void* stream) {
    RI_REQUIRE(tokens > 0 && seqs > 0 && channels > 0 && taps >= 1 && taps <= SSD_MAX_TAPS,
               "causal_conv_silu: %d tokens, %d channels, %d taps (up to %d)", tokens, channels, taps, SSD_MAX_TAPS);
    RI_REQUIRE(col0 >= 0 && col0 + channels <= stride, "causal_conv_silu: columns %d..%d of rows of %d", col0, col0 + channels, stride);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "causal_conv_silu: dtype %d", act_dtype);
    RI_REQUIRE(taps == 1 || tails, "causal_conv_silu: a convolution of %d taps keeps a tail", taps);
    hipStream_t s = (hipStream_t)stream;
    const int cy = (channels + 255) / 256;
    if (!update_tails) {
        if (act_dtype == RI_F32)
            causal_conv_silu_kernel<float><<<dim3(tokens, cy), 256, 0, s>>>(out, (const float*)proj, stride, col0, taps_w, bias, tails,
                                                                           taps, tok_seq, cu_seqlens, slots, channels);
        else
            causal_conv_silu_kernel<bf16_t><<<dim3(tokens, cy), 256, 0, s>>>(out, (const bf16_t*)proj, stride, col0, taps_w, bias,
                                                                            tails, taps, tok_seq, cu_seqlens, slots, channels);
    } else if (taps > 1) {
        if (act_dtype == RI_F32)
            conv_tails_kernel<float><<<dim3(seqs, cy), 256, 0, s>>>(tails, (const float*)proj, stride, col0, taps, cu_seqlens, slots, channels);
        else
            conv_tails_kernel<bf16_t><<<dim3(seqs, cy), 256, 0, s>>>(tails, (const bf16_t*)proj, stride, col0, taps, cu_seqlens, slots, channels);
    }
    RI_LAUNCH_CHECK("causal_conv_silu");
    return 0;
}

// ------------------------------------------------------------------ the walk
// blockDim.x = vdim * slices; thread (slice, c) holds the rows slice * RPT .. + RPT - 1 (of the state's N) of column c.
template <typename TA, int RPT>
__global__ void __launch_bounds__(1024)
ssd_scan_kernel(float* __restrict__ out, const float* __restrict__ xbc, int channels, int b_off, int c_off,
                const TA* __restrict__ proj, int stride, int z_off, int dt_off, const float* __restrict__ dt_bias,
                const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
                const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots, int heads, int groups, int n,
                int vdim, int slices) {
    extern __shared__ float lds[];
    float* bs = lds;                       // [n] B
    float* cs = bs + n;                    // [n] C
    float* xs = cs + n;                    // [vdim] x
    float* red = xs + vdim;                // [slices][vdim]
    const int seq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int c = tid % vdim, slice = tid / vdim;
    const int row0 = slice * RPT;
    const int group = h / (heads / groups);
    const int inner = heads * vdim;
    float* sp = state + (((size_t)slots[seq] * heads + h) * n) * vdim;
    float st[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) st[i] = row0 + i < n ? sp[(size_t)(row0 + i) * vdim + c] : 0.f;
    const float neg_a = -expf(a_log[h]), skip = d_skip ? d_skip[h] : 0.f, bias = dt_bias ? dt_bias[h] : 0.f;
    const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
    for (int t = t0; t < t1; ++t) {
        const float* row = xbc + (size_t)t * channels;
        __syncthreads();
        for (int e = tid; e < n; e += blockDim.x) {
            bs[e] = row[b_off + group * n + e];
            cs[e] = row[c_off + group * n + e];
        }
        if (tid < vdim) xs[tid] = row[h * vdim + tid];
        __syncthreads();
        const float raw = to_f32(proj[(size_t)t * stride + dt_off + h]) + bias;
        const float dt = raw > 20.f ? raw : log1pf(expf(raw));           // softplus: beyond 20 it is its argument to the last bit
        const float decay = expf(neg_a * dt);
        const float dx = dt * xs[c];
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int r = row0 + i;
            if (r < n) {
                st[i] = decay * st[i] + bs[r] * dx;
                part += st[i] * cs[r];
            }
        }
        red[slice * vdim + c] = part;
        __syncthreads();
        if (tid < vdim) {
            float y = 0.f;
            for (int s = 0; s < slices; ++s) y += red[s * vdim + tid];
            y += skip * xs[tid];
            const float z = to_f32(proj[(size_t)t * stride + z_off + h * vdim + tid]);
            out[(size_t)t * inner + h * vdim + tid] = y * (z / (1.f + expf(-z)));
        }
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i)
        if (row0 + i < n) sp[(size_t)(row0 + i) * vdim + c] = st[i];
}

extern "C" int ri_ssd_scan(float* out, const float* xbc, int channels, int b_off, int c_off, const void* proj, int act_dtype,
                           int stride, int z_off, int dt_off, const float* dt_bias, const float* a_log, const float* d_skip,
                           float* state, const int32_t* cu_seqlens, const int32_t* slots, int seqs, int heads, int groups,
                           int n, int vdim, void* stream) {
    RI_REQUIRE(seqs > 0 && heads > 0 && heads <= 65535 && groups > 0 && heads % groups == 0 && n >= 1 && vdim >= 1 && vdim <= 256 &&
               n <= 1024, "ssd_scan: %d sequences, %d heads in %d groups, state %d x %d", seqs, heads, groups, n, vdim);
    RI_REQUIRE(b_off >= 0 && c_off >= 0 && b_off + groups * n <= channels && c_off + groups * n <= channels && heads * vdim <= channels,
               "ssd_scan: columns %d and %d of %d channels", b_off, c_off, channels);
    RI_REQUIRE(z_off >= 0 && dt_off >= 0 && z_off + heads * vdim <= stride && dt_off + heads <= stride,
               "ssd_scan: columns %d and %d of rows of %d", z_off, dt_off, stride);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "ssd_scan: dtype %d", act_dtype);
    int slices = (n + 31) / 32;
    while (slices * 2 * vdim <= 256) slices *= 2;
    if (slices > n) slices = n;
    while (slices > 1 && slices * vdim > 1024) slices /= 2;
    const int rpt = (n + slices - 1) / slices;
    RI_REQUIRE(slices * vdim <= 1024 && rpt <= 64, "ssd_scan: a state of %d x %d does not fit a workgroup", n, vdim);
    const dim3 grid(seqs, heads);
    const int threads = slices * vdim;
    const size_t lds = ((size_t)2 * n + vdim + (size_t)slices * vdim) * sizeof(float);
    hipStream_t s = (hipStream_t)stream;
#define RI_GO(TA, RPT)                                                                                                  \
    ssd_scan_kernel<TA, RPT><<<grid, threads, lds, s>>>(out, xbc, channels, b_off, c_off, (const TA*)proj, stride, z_off, \
                                                        dt_off, dt_bias, a_log, d_skip, state, cu_seqlens, slots, heads, \
                                                        groups, n, vdim, slices)
#define RI_BY_ROWS(TA)                                                                                                  \
    if (rpt <= 8) RI_GO(TA, 8); else if (rpt <= 16) RI_GO(TA, 16); else if (rpt <= 32) RI_GO(TA, 32); else RI_GO(TA, 64)
    if (act_dtype == RI_F32) { RI_BY_ROWS(float); } else { RI_BY_ROWS(bf16_t); }
#undef RI_BY_ROWS
#undef RI_GO
    RI_LAUNCH_CHECK("ssd_scan");
    return 0;
}

// ------------------------------------------------------------------ the walk, a wavefront on 16 columns
// States of up to 128 rows: a wavefront owns 16 columns of one (sequence, head), its lanes four slices of the rows of a
// column each (8 columns and eight slices for states above 64 rows), the rows in registers; a token's sum over the rows is the lane's own sum (four partial sums, so that no
// addition waits for the one before) and two exchanges between the lanes of a column.  A workgroup is four wavefronts
// on columns of their own, which share the tokens staged in LDS in blocks of SSD_BLOCK (B, C, x, the step size and decay, z), the next block's loads asked
// for before the block in work is computed.  The order of a token's additions is fixed by the sizes alone.
#define SSD_BLOCK 8
#define SSD_WAVES 4          // wavefronts of a workgroup: they share the staged tokens, each on columns of its own

template <typename TA, int RPL, int SL>                       // RPL: rows a lane holds, a multiple of 4; SL: slices of rows, 4 or 8
__global__ void __launch_bounds__(64 * SSD_WAVES)
ssd_scan_cols_kernel(float* __restrict__ out, const float* __restrict__ xbc, int channels, int b_off, int c_off,
                     const TA* __restrict__ proj, int stride, int z_off, int dt_off, const float* __restrict__ dt_bias,
                     const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
                     const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots, int heads, int groups, int n,
                     int vdim) {
    // COLS: columns of a wavefront; NC: of the workgroup; TPP: tokens whose x and z one pass of the workgroup's threads fetches
    constexpr int ROWS = SL * RPL, COLS = 64 / SL, NC = COLS * SSD_WAVES, THREADS = 64 * SSD_WAVES, TPP = THREADS / NC,
                  PASSES = SSD_BLOCK / TPP;
    __shared__ __attribute__((aligned(16))) float bs[2][SSD_BLOCK][ROWS];
    __shared__ __attribute__((aligned(16))) float cs[2][SSD_BLOCK][ROWS];
    __shared__ float xs[2][SSD_BLOCK][NC];
    __shared__ float zs[2][SSD_BLOCK][NC];
    __shared__ float dts[2][SSD_BLOCK], decays[2][SSD_BLOCK];
    const int seq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane % COLS, slice = lane / COLS, row0 = slice * RPL;
    const int wcol = wave * COLS + col;                       // the lane's column among the workgroup's
    const int c = blockIdx.z * NC + wcol;
    const bool has_col = c < vdim;
    const int cc = has_col ? c : vdim - 1;                    // a column pulled back inside the head: loads are issued anyway
    const int group = h / (heads / groups), inner = heads * vdim;
    float* sp = state + (((size_t)slots[seq] * heads + h) * n) * vdim + cc;
    float st[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) st[i] = row0 + i < n ? sp[(size_t)(row0 + i) * vdim] : 0.f;
    const float neg_a = -expf(a_log[h]), skip = d_skip ? d_skip[h] : 0.f, bias = dt_bias ? dt_bias[h] : 0.f;
    const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
    constexpr int PER = (2 * SSD_BLOCK * ROWS + THREADS - 1) / THREADS;     // B and C elements of a block a thread stages
    const int vcol = min((int)blockIdx.z * NC + tid % NC, vdim - 1), vtok = tid / NC;      // the thread's place in a pass over x and z

    float pre_bc[PER], pre_x[PASSES], pre_z[PASSES], pre_raw = 0.f;
    auto fetch = [&](int tb) {                                // a block's loads, into registers
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = tid + i * THREADS;                  // (which, token, row)
            const int r = e % ROWS, tt = (e / ROWS) % SSD_BLOCK, which = e / (ROWS * SSD_BLOCK);
            const int t = min(tb + tt, t1 - 1);
            pre_bc[i] = (r < n && which < 2) ? xbc[(size_t)t * channels + (which ? c_off : b_off) + group * n + r] : 0.f;
        }
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {                 // x and z of the block's tokens for this wavefront's columns
            const int t = min(tb + ps * TPP + vtok, t1 - 1);
            pre_x[ps] = xbc[(size_t)t * channels + h * vdim + vcol];
            pre_z[ps] = to_f32(proj[(size_t)t * stride + z_off + h * vdim + vcol]);
        }
        if (tid < SSD_BLOCK) pre_raw = to_f32(proj[(size_t)min(tb + tid, t1 - 1) * stride + dt_off + h]);
    };
    auto stage = [&](int buf) {                               // ... and from there into LDS
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = tid + i * THREADS;
            const int r = e % ROWS, tt = (e / ROWS) % SSD_BLOCK, which = e / (ROWS * SSD_BLOCK);
            if (which == 0) bs[buf][tt][r] = pre_bc[i];
            else if (which == 1) cs[buf][tt][r] = pre_bc[i];
        }
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            xs[buf][ps * TPP + vtok][tid % NC] = pre_x[ps];
            zs[buf][ps * TPP + vtok][tid % NC] = pre_z[ps];
        }
        if (tid < SSD_BLOCK) {
            const float raw = pre_raw + bias;
            const float dt = raw > 20.f ? raw : log1pf(expf(raw));       // softplus: beyond 20 it is its argument to the last bit
            dts[buf][tid] = dt;
            decays[buf][tid] = expf(neg_a * dt);
        }
    };
    if (t0 < t1) {
        fetch(t0);
        stage(0);
    }
    __syncthreads();
    int buf = 0;
    for (int tb = t0; tb < t1; tb += SSD_BLOCK, buf ^= 1) {
        const bool more = tb + SSD_BLOCK < t1;
        if (more) {
            fetch(tb + SSD_BLOCK);
        }
        const int count = min(SSD_BLOCK, t1 - tb);
        float part[SSD_BLOCK];                                // the lane's share of each token's sum: the exchanges wait for the block's end,
#pragma unroll                                                // so that no token waits for the one before it
        for (int tt = 0; tt < SSD_BLOCK; ++tt) {
            part[tt] = 0.f;
            if (tt < count) {
                const float decay = decays[buf][tt];
                const float dx = dts[buf][tt] * xs[buf][tt][wcol];
                float y0 = 0.f, y1 = 0.f, y2 = 0.f, y3 = 0.f;
#pragma unroll
                for (int i = 0; i < RPL; i += 4) {
                    const float4 b4 = *reinterpret_cast<const float4*>(&bs[buf][tt][row0 + i]);
                    const float4 c4 = *reinterpret_cast<const float4*>(&cs[buf][tt][row0 + i]);
                    st[i] = decay * st[i] + b4.x * dx;             y0 += st[i] * c4.x;
                    st[i + 1] = decay * st[i + 1] + b4.y * dx;     y1 += st[i + 1] * c4.y;
                    st[i + 2] = decay * st[i + 2] + b4.z * dx;     y2 += st[i + 2] * c4.z;
                    st[i + 3] = decay * st[i + 3] + b4.w * dx;     y3 += st[i + 3] * c4.w;
                }
                part[tt] = (y0 + y1) + (y2 + y3);
            }
        }
#pragma unroll
        for (int tt = 0; tt < SSD_BLOCK; ++tt) {
            float y = part[tt];
            if (SL == 8) y += __shfl_xor(y, 8, RI_WAVE);      // the slices of a column
            y += __shfl_xor(y, 16, RI_WAVE);
            y += __shfl_xor(y, 32, RI_WAVE);
            if (tt < count && has_col && slice == 0) {
                y += skip * xs[buf][tt][wcol];
                const float z = zs[buf][tt][wcol];
                out[(size_t)(tb + tt) * inner + h * vdim + c] = y * (z / (1.f + expf(-z)));
            }
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    }
    if (has_col) {
#pragma unroll
        for (int i = 0; i < RPL; ++i)
            if (row0 + i < n) sp[(size_t)(row0 + i) * vdim] = st[i];
    }
}

extern "C" int ri_ssd_scan_cols_fits(int n, int vdim) { return n >= 1 && n <= 128 && vdim >= 1; }

extern "C" int ri_ssd_scan_cols(float* out, const float* xbc, int channels, int b_off, int c_off, const void* proj, int act_dtype,
                                int stride, int z_off, int dt_off, const float* dt_bias, const float* a_log, const float* d_skip,
                                float* state, const int32_t* cu_seqlens, const int32_t* slots, int seqs, int heads, int groups,
                                int n, int vdim, void* stream) {
    RI_REQUIRE(seqs > 0 && heads > 0 && heads <= 65535 && groups > 0 && heads % groups == 0 && ri_ssd_scan_cols_fits(n, vdim),
               "ssd_scan_cols: %d sequences, %d heads in %d groups, state %d x %d", seqs, heads, groups, n, vdim);
    RI_REQUIRE(b_off >= 0 && c_off >= 0 && b_off + groups * n <= channels && c_off + groups * n <= channels && heads * vdim <= channels,
               "ssd_scan_cols: columns %d and %d of %d channels", b_off, c_off, channels);
    RI_REQUIRE(z_off >= 0 && dt_off >= 0 && z_off + heads * vdim <= stride && dt_off + heads <= stride,
               "ssd_scan_cols: columns %d and %d of rows of %d", z_off, dt_off, stride);
    RI_REQUIRE(act_dtype == RI_F32 || act_dtype == RI_BF16, "ssd_scan_cols: dtype %d", act_dtype);
    const int cols = (n > 64 ? 8 : 16) * SSD_WAVES;
    const dim3 grid(seqs, heads, (vdim + cols - 1) / cols);
    RI_REQUIRE(grid.z <= 65535, "ssd_scan_cols: heads of %d channels", vdim);
    hipStream_t s = (hipStream_t)stream;
#define RI_GO(TA, RPL, SL)                                                                                              \
    ssd_scan_cols_kernel<TA, RPL, SL><<<grid, 64 * SSD_WAVES, 0, s>>>(out, xbc, channels, b_off, c_off, (const TA*)proj, stride, z_off,  \
                                                      dt_off, dt_bias, a_log, d_skip, state, cu_seqlens, slots, heads,   \
                                                      groups, n, vdim)
#define RI_BY_ROWS(TA)                                                                                                  \
    if (n <= 16) RI_GO(TA, 4, 4); else if (n <= 32) RI_GO(TA, 8, 4); else if (n <= 64) RI_GO(TA, 16, 4); else RI_GO(TA, 16, 8)
    if (act_dtype == RI_F32) { RI_BY_ROWS(float); } else { RI_BY_ROWS(bf16_t); }
#undef RI_BY_ROWS
#undef RI_GO
    RI_LAUNCH_CHECK("ssd_scan_cols");
    return 0;
}

// ------------------------------------------------------------------ the norm in parts
template <typename TO>
__global__ void __launch_bounds__(256)
group_rms_norm_kernel(TO* __restrict__ out, const float* __restrict__ x, const float* __restrict__ gain, float eps, int width,
                      int part) {
    __shared__ float scratch[16];
    const size_t at = (size_t)blockIdx.x * width + (size_t)blockIdx.y * part;
    float ss = 0.f;
    for (int d = threadIdx.x; d < part; d += 256) ss += x[at + d] * x[at + d];
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
    for (int d = threadIdx.x; d < part; d += 256)
        from_f32(out + at + d, x[at + d] * inv * (gain ? gain[blockIdx.y * part + d] : 1.f));
}

extern "C" int ri_group_rms_norm(void* out, int out_dtype, const float* x, const float* gain, float eps, int rows, int width,
                                 int parts, void* stream) {
    RI_REQUIRE(rows > 0 && width > 0 && parts >= 1 && parts <= 65535 && width % parts == 0, "group_rms_norm: %d rows of %d in %d parts",
               rows, width, parts);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "group_rms_norm: dtype %d", out_dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, parts);
    if (out_dtype == RI_F32) group_rms_norm_kernel<float><<<grid, 256, 0, s>>>((float*)out, x, gain, eps, width, width / parts);
    else group_rms_norm_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out, x, gain, eps, width, width / parts);
    RI_LAUNCH_CHECK("group_rms_norm");
    return 0;
}
