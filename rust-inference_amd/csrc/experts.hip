// A mixture of experts: the router's choice and weights, and the experts' activation.
//
// Router: s = sigmoid(z) of the float32 logits; the choice is by s + correction, the weights are the chosen
// experts' s over their sum.  The experts themselves are products: every expert's gate and up branch side by side
// in one matrix, [experts, 2, ff] rows, and every expert's down matrix side by side along K, so that the weighted
// sum over the chosen experts is the one product's sum over K, with the weight of an expert that was not chosen
// being zero.
#include "api.h"
#include "common.h"

#define EXPERTS_MAX 1024

// One wavefront a token.  The router's outputs are `outs` = experts + identity experts (an identity expert hands the
// token's own row on, times its weight; it has no matrices and is the business of whoever adds the experts up).
//   scores:  s = sigmoid(z) or softmax(z) over all outputs (float32; the softmax with its maximum taken off);
//   choice:  by s + correction; with groups, the outputs form `groups` equal runs of neighbours, a group's score is
//            its largest choice score, and only outputs of the `keep` best groups can be chosen (the others count as
//            minus infinity); the `top` largest, the lower index on a tie;
//   weights: the chosen outputs' s, divided by their sum (+ 1e-20) when `normalize`.
// z rows have z_stride >= outs columns; with `extra`, extra[t, 0] is the sum of the weights of the identity experts
// chosen and extra[t, 1] = sigmoid(z[t, outs]), the gate of an expert that every token uses, whose logit rides as one
// more row of the router's matrix.
#define ROUTE_SIGMOID 0
#define ROUTE_SOFTMAX 1
__global__ void __launch_bounds__(64)
experts_route_kernel(int32_t* __restrict__ ids, float* __restrict__ weights, float* __restrict__ dense,
                     float* __restrict__ extra, const float* __restrict__ z, int z_stride,
                     const float* __restrict__ correction, int outs, int experts, int top, int kind, int normalize,
                     int groups, int keep) {
    __shared__ float sc[EXPERTS_MAX], ch[EXPERTS_MAX], gbest[EXPERTS_MAX];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* zt = z + (size_t)t * z_stride;
    float* dt = dense + (size_t)t * outs;
    if (kind == ROUTE_SOFTMAX) {
        float m = -INFINITY;
        for (int e = lane; e < outs; e += RI_WAVE) m = fmaxf(m, zt[e]);
        m = wave_max(m);
        float sum = 0.f;
        for (int e = lane; e < outs; e += RI_WAVE) {
            const float v = expf(zt[e] - m);
            sc[e] = v;
            sum += v;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < outs; e += RI_WAVE) sc[e] = sc[e] / sum;
    } else {
        for (int e = lane; e < outs; e += RI_WAVE) sc[e] = 1.f / (1.f + expf(-zt[e]));
    }
    for (int e = lane; e < outs; e += RI_WAVE) {
        ch[e] = sc[e] + correction[e];
        dt[e] = 0.f;
    }
    __syncthreads();
    if (groups > 1 && keep < groups) {
        const int per = outs / groups;
        for (int g = lane; g < groups; g += RI_WAVE) {
            float best = -INFINITY;
            for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, ch[e]);
            gbest[g] = best;
        }
        __syncthreads();
        for (int g = lane; g < groups; g += RI_WAVE) {
            int ahead = 0;                                    // groups that come before this one: better, or as good and earlier
            for (int o = 0; o < groups; ++o) ahead += gbest[o] > gbest[g] || (gbest[o] == gbest[g] && o < g);
            if (ahead >= keep)
                for (int e = g * per; e < (g + 1) * per; ++e) ch[e] = -INFINITY;
        }
        __syncthreads();
    }
    float sum = 0.f, identity = 0.f;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float best_choice = 0.f;
        for (int e = lane; e < outs; e += RI_WAVE) {
            const float c = ch[e];
            if (c == -INFINITY && best >= 0) continue;
            if (best < 0 || c > best_choice) { best = e; best_choice = c; }
        }
        // the wavefront's best: the larger choice score, the lower index on a tie; lanes without an output lose
        for (int m = RI_WAVE / 2; m > 0; m >>= 1) {
            const int ob = __shfl_xor(best, m, RI_WAVE);
            const float oc = __shfl_xor(best_choice, m, RI_WAVE);
            if (ob >= 0 && (best < 0 || oc > best_choice || (oc == best_choice && ob < best))) { best = ob; best_choice = oc; }
        }
        const float w = sc[best];
        __syncthreads();
        if (lane == 0) {
            ids[(size_t)t * top + k] = best;
            weights[(size_t)t * top + k] = w;
            ch[best] = -INFINITY;
        }
        __syncthreads();
        sum += w;
    }
    const float inv = normalize ? 1.f / (sum + 1e-20f) : 1.f;
    if (lane == 0) {
        for (int k = 0; k < top; ++k) {
            const float w = weights[(size_t)t * top + k] * inv;
            const int e = ids[(size_t)t * top + k];
            weights[(size_t)t * top + k] = w;
            dt[e] = w;
            if (e >= experts) identity += w;
        }
        if (extra) {
            extra[(size_t)t * 2] = identity;
            extra[(size_t)t * 2 + 1] = z_stride > outs ? 1.f / (1.f + expf(-zt[outs])) : 0.f;
        }
    }
}

// An expert's activation from its gate and up branches.  limit > 0: g = min(gate, limit), u = clamp(up, -limit,
// limit), g sigmoid(1.702 g) (u + 1).  limit <= 0: the plain gated form silu(gate) * up.
__device__ __forceinline__ float expert_act(float gate, float up, float limit) {
    if (limit > 0.f) {
        const float a = fminf(gate, limit);
        const float u = fminf(fmaxf(up, -limit), limit);
        return a / (1.f + expf(-1.702f * a)) * (u + 1.f);
    }
    return gate / (1.f + expf(-gate)) * up;
}

template <typename T>
__global__ void __launch_bounds__(256)
experts_activate_kernel(T* __restrict__ out, const T* __restrict__ gu, const float* __restrict__ dense, int dense_stride,
                        int experts, int ff, float limit) {
    const int t = blockIdx.x, e = blockIdx.y;
    const float w = dense ? dense[(size_t)t * dense_stride + e] : 1.f;   // no weights: every row is of its expert
    T* o = out + ((size_t)t * experts + e) * ff;
    const T* g = gu + ((size_t)t * experts + e) * 2 * ff;
    for (int i = threadIdx.x; i < ff; i += blockDim.x) {
        float v = 0.f;
        if (w != 0.f) {
            v = w * expert_act(to_f32(g[i]), to_f32(g[ff + i]), limit);
        }
        from_f32(o + i, v);
    }
}

// ---- a few tokens: only the chosen experts' rows are read
// One wavefront an (assignment, row i): the gate row i and the up row i of the assignment's expert against the
// token's row, 16 bytes a lane at a time, then the activation times the router's weight.  gu: [experts, 2, ff, dim]
// rows (gate then up); act: [tokens * top, ff].
__global__ void __launch_bounds__(256)
experts_gate_up_rows_kernel(bf16_t* __restrict__ act, const bf16_t* __restrict__ x, const bf16_t* __restrict__ gu,
                            const int32_t* __restrict__ ids, const float* __restrict__ weights, int top, int ff, int dim,
                            float limit, int experts) {
    const int lane = threadIdx.x & 63, i = blockIdx.x * 4 + (threadIdx.x >> 6), pair = blockIdx.y;
    if (i >= ff) return;                                      // (whole wavefronts)
    const int e = ids[pair];
    if (e >= experts) return;                                 // an identity expert has no rows: the sum below adds the token's own
    const bf16_t* xr = x + (size_t)(pair / top) * dim;
    const bf16_t* gr = gu + ((size_t)e * 2 * ff + i) * dim;
    const bf16_t* ur = gr + (size_t)ff * dim;
    float g = 0.f, u = 0.f;
    for (int c = lane * 8; c < dim; c += 512) {
        const uint4 a = load_stream16(gr + c), b = load_stream16(ur + c), v = *reinterpret_cast<const uint4*>(xr + c);
        const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w}, vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float x0 = __uint_as_float(vw[k] << 16), x1 = __uint_as_float(vw[k] & 0xFFFF0000u);
            g += __uint_as_float(aw[k] << 16) * x0 + __uint_as_float(aw[k] & 0xFFFF0000u) * x1;
            u += __uint_as_float(bw[k] << 16) * x0 + __uint_as_float(bw[k] & 0xFFFF0000u) * x1;
        }
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) {
        // the products' results pass through bfloat16, as they do where the products are kernels of their own
        act[(size_t)pair * ff + i] = f32_to_bf16(weights[pair] * expert_act(bf16_to_f32(f32_to_bf16(g)),
                                                                             bf16_to_f32(f32_to_bf16(u)), limit));
    }
}

// One wavefront an output row n of a token: the sum over the token's chosen experts, in the order chosen, of the
// expert's down row n against the assignment's activations.  down: [dim, experts * ff] (the experts side by side
// along a row); out: float32 [tokens, dim].
__global__ void __launch_bounds__(256)
experts_down_rows_kernel(float* __restrict__ out, const bf16_t* __restrict__ act, const bf16_t* __restrict__ down,
                         const int32_t* __restrict__ ids, int top, int ff, int dim, int experts,
                         const bf16_t* __restrict__ x, const float* __restrict__ weights) {
    const int lane = threadIdx.x & 63, n = blockIdx.x * 4 + (threadIdx.x >> 6), t = blockIdx.y;
    if (n >= dim) return;
    float acc = 0.f, own = 0.f;
    for (int k = 0; k < top; ++k) {
        const int pair = t * top + k;
        if (ids[pair] >= experts) {                           // an identity expert: the token's own row times the weight
            own += weights[pair] * bf16_to_f32(x[(size_t)t * dim + n]);
            continue;
        }
        const bf16_t* wr = down + (size_t)n * experts * ff + (size_t)ids[pair] * ff;
        const bf16_t* ar = act + (size_t)pair * ff;
        for (int c = lane * 8; c < ff; c += 512) {
            const uint4 a = load_stream16(wr + c), v = *reinterpret_cast<const uint4*>(ar + c);
            const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc += __uint_as_float(aw[j] << 16) * __uint_as_float(vw[j] << 16)
                     + __uint_as_float(aw[j] & 0xFFFF0000u) * __uint_as_float(vw[j] & 0xFFFF0000u);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) out[(size_t)t * dim + n] = acc + own;
}

extern "C" int ri_experts_few_tokens(float* out, void* act, const void* x, const void* gu, const void* down,
                                     const int32_t* ids, const float* weights, int tokens, int experts, int top, int ff,
                                     int dim, float limit, void* stream) {
    RI_REQUIRE(tokens > 0 && experts >= 1 && top >= 1, "experts_few_tokens: %d tokens, %d of %d experts", tokens, top, experts);
    RI_REQUIRE(ff >= 8 && ff % 8 == 0 && dim >= 8 && dim % 8 == 0, "experts_few_tokens: sizes %d and %d must be multiples of 8", ff, dim);
    RI_REQUIRE((long)tokens * top <= 65535 && tokens <= 65535, "experts_few_tokens: %d tokens exceed one launch", tokens);
    hipStream_t s = (hipStream_t)stream;
    experts_gate_up_rows_kernel<<<dim3((ff + 3) / 4, tokens * top), 256, 0, s>>>(
        (bf16_t*)act, (const bf16_t*)x, (const bf16_t*)gu, ids, weights, top, ff, dim, limit, experts);
    RI_LAUNCH_CHECK("experts_few_tokens (gate and up)");
    experts_down_rows_kernel<<<dim3((dim + 3) / 4, tokens), 256, 0, s>>>(out, (const bf16_t*)act, (const bf16_t*)down, ids,
                                                                       top, ff, dim, experts, (const bf16_t*)x, weights);
    RI_LAUNCH_CHECK("experts_few_tokens (down)");
    return 0;
}

// ---- many tokens: the assignments sorted by expert, so that every expert's tokens are rows side by side
// One workgroup an expert: it walks all assignments in order and numbers its own, so that the order inside an
// expert is the order of the tokens whatever ran first.
__global__ void __launch_bounds__(256)
experts_rank_kernel(int32_t* __restrict__ rank, int32_t* __restrict__ counts, const int32_t* __restrict__ ids, int pairs) {
    __shared__ int wave_count[4];
    const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int before = 0;
    for (int base = 0; base < pairs; base += 256) {
        const int p = base + threadIdx.x;
        const bool mine = p < pairs && ids[p] == e;
        const unsigned long long votes = __ballot(mine);
        if (lane == 0) wave_count[wave] = __builtin_popcountll(votes);
        __syncthreads();
        int ahead = __builtin_popcountll(votes & ((1ull << lane) - 1ull)), all = 0;
        for (int w = 0; w < 4; ++w) {
            if (w < wave) ahead += wave_count[w];
            all += wave_count[w];
        }
        if (mine) rank[p] = before + ahead;
        before += all;
        __syncthreads();
    }
    if (threadIdx.x == 0) counts[e] = before;
}

// offsets[e]: where expert e's rows begin (offsets[experts]: the number of assignments); dest[p]: the row of
// assignment p.  One workgroup.
__global__ void __launch_bounds__(256)
experts_place_kernel(int32_t* __restrict__ dest, int32_t* __restrict__ offsets, const int32_t* __restrict__ rank,
                     const int32_t* __restrict__ counts, const int32_t* __restrict__ ids, int pairs, int experts) {
    __shared__ int start[EXPERTS_MAX + 1];
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            start[e] = at;
            at += counts[e];
        }
        start[experts] = at;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= experts; e += blockDim.x) offsets[e] = start[e];
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) dest[p] = start[ids[p]] + rank[p];
}

// rows[dest[p], :] = x[p / top, :], 16 bytes a thread at a time (dim a multiple of 8 bfloat16).
__global__ void __launch_bounds__(256)
experts_gather_kernel(bf16_t* __restrict__ rows, const bf16_t* __restrict__ x, const int32_t* __restrict__ dest, int top,
                      int dim) {
    const int p = blockIdx.x;
    const uint4* from = reinterpret_cast<const uint4*>(x + (size_t)(p / top) * dim);
    uint4* to = reinterpret_cast<uint4*>(rows + (size_t)dest[p] * dim);
    for (int c = threadIdx.x; c < dim / 8; c += blockDim.x) to[c] = from[c];
}

// out[t, :] = sum over the token's assignments k, in order, of weights[t, k] * y[dest[t * top + k], :], in float32.
// VEC: 16 bytes of y a thread at a time (dim a multiple of 8).
template <bool VEC>
__global__ void __launch_bounds__(256)
experts_combine_kernel(float* __restrict__ out, const bf16_t* __restrict__ y, const int32_t* __restrict__ dest,
                       const float* __restrict__ weights, int top, int dim) {
    const int t = blockIdx.x;
    if (VEC) {
        for (int c = threadIdx.x * 8; c < dim; c += blockDim.x * 8) {
            float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < top; ++k) {
                const float w = weights[(size_t)t * top + k];
                const uint4 v = *reinterpret_cast<const uint4*>(y + (size_t)dest[(size_t)t * top + k] * dim + c);
                const uint32_t vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[2 * j] += w * __uint_as_float(vw[j] << 16);
                    acc[2 * j + 1] += w * __uint_as_float(vw[j] & 0xFFFF0000u);
                }
            }
            float4* to = reinterpret_cast<float4*>(out + (size_t)t * dim + c);
            to[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
            to[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
        }
        return;
    }
    for (int c = threadIdx.x; c < dim; c += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k)
            acc += weights[(size_t)t * top + k] * bf16_to_f32(y[(size_t)dest[(size_t)t * top + k] * dim + c]);
        out[(size_t)t * dim + c] = acc;
    }
}

extern "C" int ri_experts_sort(int32_t* dest, int32_t* offsets, int32_t* rank, int32_t* counts, const int32_t* ids,
                               int pairs, int experts, void* stream) {
    RI_REQUIRE(pairs > 0 && experts >= 1 && experts <= EXPERTS_MAX, "experts_sort: %d assignments to %d experts", pairs, experts);
    hipStream_t s = (hipStream_t)stream;
    experts_rank_kernel<<<experts, 256, 0, s>>>(rank, counts, ids, pairs);
    RI_LAUNCH_CHECK("experts_sort (rank)");
    experts_place_kernel<<<1, 256, 0, s>>>(dest, offsets, rank, counts, ids, pairs, experts);
    RI_LAUNCH_CHECK("experts_sort (place)");
    return 0;
}

extern "C" int ri_experts_gather(void* rows, const void* x, const int32_t* dest, int pairs, int top, int dim, void* stream) {
    RI_REQUIRE(pairs > 0 && top >= 1 && pairs % top == 0 && dim >= 8 && dim % 8 == 0,
               "experts_gather: %d assignments, %d a token, rows of %d", pairs, top, dim);
    experts_gather_kernel<<<pairs, 256, 0, (hipStream_t)stream>>>((bf16_t*)rows, (const bf16_t*)x, dest, top, dim);
    RI_LAUNCH_CHECK("experts_gather");
    return 0;
}

extern "C" int ri_experts_combine(float* out, const void* y, const int32_t* dest, const float* weights, int tokens, int top,
                                  int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && top >= 1 && dim >= 1, "experts_combine: %d tokens, %d a token, rows of %d", tokens, top, dim);
    if (dim % 8 == 0 && (uintptr_t)y % 16 == 0 && (uintptr_t)out % 16 == 0)
        experts_combine_kernel<true><<<tokens, 256, 0, (hipStream_t)stream>>>(out, (const bf16_t*)y, dest, weights, top, dim);
    else
        experts_combine_kernel<false><<<tokens, 256, 0, (hipStream_t)stream>>>(out, (const bf16_t*)y, dest, weights, top, dim);
    RI_LAUNCH_CHECK("experts_combine");
    return 0;
}

extern "C" int ri_experts_route_general(int32_t* ids, float* weights, float* dense, float* extra, const float* z, int z_stride,
                                        const float* correction, int tokens, int outs, int experts, int top, int kind,
                                        int normalize, int groups, int keep, void* stream) {
    RI_REQUIRE(tokens > 0 && experts >= 0 && experts <= outs && outs >= 1 && outs <= EXPERTS_MAX && top >= 1 && top <= outs,
               "experts_route: %d tokens, the %d best of %d outputs (%d experts; at most %d)", tokens, top, outs, experts, EXPERTS_MAX);
    RI_REQUIRE(kind == ROUTE_SIGMOID || kind == ROUTE_SOFTMAX, "experts_route: score kind %d", kind);
    RI_REQUIRE(groups >= 1 && outs % groups == 0 && keep >= 1 && keep <= groups && (long)keep * (outs / groups) >= top,
               "experts_route: %d outputs in %d groups of which %d stay, for the %d best", outs, groups, keep, top);
    RI_REQUIRE(z_stride >= outs, "experts_route: logit rows of %d for %d outputs", z_stride, outs);
    experts_route_kernel<<<tokens, 64, 0, (hipStream_t)stream>>>(ids, weights, dense, extra, z, z_stride, correction, outs,
                                                                  experts, top, kind, normalize, groups, keep);
    RI_LAUNCH_CHECK("experts_route");
    return 0;
}

extern "C" int ri_experts_route(int32_t* ids, float* weights, float* dense, const float* z, const float* correction,
                                int tokens, int experts, int top, void* stream) {
    return ri_experts_route_general(ids, weights, dense, nullptr, z, experts, correction, tokens, experts, experts, top,
                                    ROUTE_SIGMOID, 1, 1, 1, stream);
}

extern "C" int ri_experts_activate_strided(void* out, const void* gu, int dtype, const float* dense, int dense_stride,
                                           int tokens, int experts, int ff, float limit, void* stream) {
    RI_REQUIRE(!dense || dense_stride >= experts, "experts_activate: weight rows of %d for %d experts", dense_stride, experts);
    RI_REQUIRE(tokens > 0 && experts >= 1 && experts <= 65535 && ff >= 1, "experts_activate: %d tokens, %d experts of %d",
               tokens, experts, ff);
    RI_REQUIRE(dtype == RI_F32 || dtype == RI_BF16, "experts_activate: dtype %d", dtype);
    const dim3 grid(tokens, experts);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == RI_F32)
        experts_activate_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)gu, dense, dense_stride, experts, ff, limit);
    else
        experts_activate_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)gu, dense, dense_stride, experts, ff, limit);
    RI_LAUNCH_CHECK("experts_activate");
    return 0;
}

extern "C" int ri_experts_activate(void* out, const void* gu, int dtype, const float* dense, int tokens, int experts,
                                   int ff, float limit, void* stream) {
    return ri_experts_activate_strided(out, gu, dtype, dense, experts, tokens, experts, ff, limit, stream);
}

// What a mixture of experts adds beside its routed experts' weighted sum, row by row, in float32:
//   out[t] = routed[t] + own[t] * x[t] + gate[t] * shared[t]
// own: the weight of the token's own row (the identity experts it chose), gate: the weight of an expert that every
// token uses; both are columns of extra [tokens, 2].  routed may come as parts of a split product, added in order;
// x and shared may be absent.
template <typename TX, typename TS>
__global__ void __launch_bounds__(256)
experts_finish_kernel(float* __restrict__ out, const float* __restrict__ routed, int parts, size_t part_stride,
                      const TX* __restrict__ x, const TS* __restrict__ shared, int shared_parts,
                      const float* __restrict__ extra, int dim) {
    const size_t at = (size_t)blockIdx.x * dim;
    const float own = extra[(size_t)blockIdx.x * 2], gate = extra[(size_t)blockIdx.x * 2 + 1];
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float v = routed[at + d];
        for (int p = 1; p < parts; ++p) v += routed[p * part_stride + at + d];
        if (x) v += own * to_f32(x[at + d]);
        if (shared) {
            float sv = to_f32(shared[at + d]);
            for (int p = 1; p < shared_parts; ++p) sv += to_f32(shared[p * part_stride + at + d]);
            v += gate * sv;
        }
        out[at + d] = v;
    }
}

// Rows whose width is a multiple of 4: a thread takes four neighbours of a row, a workgroup 1,024 columns, so that a
// step of one token is many short workgroups and not one that walks the row.
__device__ __forceinline__ float4 fin_ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 fin_ld4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16),
                       __uint_as_float(w.y & 0xFFFF0000u));
}

template <typename TX, typename TS>
__global__ void __launch_bounds__(256)
experts_finish_vec_kernel(float* __restrict__ out, const float* __restrict__ routed, int parts, size_t part_stride,
                          const TX* __restrict__ x, const TS* __restrict__ shared, int shared_parts,
                          const float* __restrict__ extra, int dim) {
    const int d = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (d >= dim) return;
    const size_t at = (size_t)blockIdx.x * dim + d;
    const float own = extra[(size_t)blockIdx.x * 2], gate = extra[(size_t)blockIdx.x * 2 + 1];
    float4 v = fin_ld4(routed + at);
    for (int p = 1; p < parts; ++p) {
        const float4 w = fin_ld4(routed + p * part_stride + at);
        v = make_float4(v.x + w.x, v.y + w.y, v.z + w.z, v.w + w.w);
    }
    if (x) {
        const float4 w = fin_ld4(x + at);
        v = make_float4(v.x + own * w.x, v.y + own * w.y, v.z + own * w.z, v.w + own * w.w);
    }
    if (shared) {
        float4 sv = fin_ld4(shared + at);
        for (int p = 1; p < shared_parts; ++p) {
            const float4 w = fin_ld4(shared + p * part_stride + at);
            sv = make_float4(sv.x + w.x, sv.y + w.y, sv.z + w.z, sv.w + w.w);
        }
        v = make_float4(v.x + gate * sv.x, v.y + gate * sv.y, v.z + gate * sv.z, v.w + gate * sv.w);
    }
    *reinterpret_cast<float4*>(out + at) = v;
}

extern "C" int ri_experts_finish(float* out, const float* routed, int parts, const void* x, int x_dtype, const void* shared,
                                 int shared_dtype, int shared_parts, const float* extra, int tokens, int dim, void* stream) {
    RI_REQUIRE(tokens > 0 && dim > 0 && parts >= 1 && shared_parts >= 1 && extra && routed, "experts_finish: %d tokens of %d", tokens, dim);
    RI_REQUIRE((x_dtype == RI_F32 || x_dtype == RI_BF16) && (shared_dtype == RI_F32 || shared_dtype == RI_BF16),
               "experts_finish: dtypes %d and %d", x_dtype, shared_dtype);
    RI_REQUIRE(shared_parts == 1 || shared_dtype == RI_F32, "experts_finish: parts of a product are float32");
    hipStream_t s = (hipStream_t)stream;
    const size_t stride = (size_t)tokens * dim;
    const dim3 vgrid(tokens, (dim / 4 + 255) / 256);
#define RI_GO(TX, TS)                                                                                                   \
    if (dim % 4 == 0 && vgrid.y <= 65535)                                                                               \
        experts_finish_vec_kernel<TX, TS><<<vgrid, 256, 0, s>>>(out, routed, parts, stride, (const TX*)x,                 \
                                                                (const TS*)shared, shared_parts, extra, dim);            \
    else                                                                                                                \
        experts_finish_kernel<TX, TS><<<tokens, 256, 0, s>>>(out, routed, parts, stride, (const TX*)x,                    \
                                                             (const TS*)shared, shared_parts, extra, dim)
    if (x_dtype == RI_F32) { if (shared_dtype == RI_F32) RI_GO(float, float); else RI_GO(float, bf16_t); }
    else                   { if (shared_dtype == RI_F32) RI_GO(bf16_t, float); else RI_GO(bf16_t, bf16_t); }
#undef RI_GO
    RI_LAUNCH_CHECK("experts_finish");
    return 0;
}
