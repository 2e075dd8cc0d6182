// A mixture of experts: the router's choice per token and the chosen experts' products.
//
// Router (float arithmetic): s = softmax(z) over all E experts; the experts form `groups`
// equal groups of neighbours, a group's score is its largest s, only experts of the `keep`
// best groups can be chosen, and of those the `top` with the largest s are; a chosen expert's
// weight is its s over the sum of the chosen s (+ weight_eps).  Ties go to the lower index.
//
// Products, one (token, chosen expert) pair at a time: h = act(W_up[e] x), and
// y = sum_k weight_k W_down[e_k] h_k in the order of the choice.  Every output element is one
// chain of multiply-adds over its own inputs, so a token's result does not depend on what
// else the step holds.  These kernels serve the float32 engine and the steps of few rows;
// the weights of an expert are stacked: W_up [E, F, D], W_down [E, D, F].
#include "common.h"

#define RE_MAX_PER_LANE 16          // experts per lane of the router's wave: E <= 1024

// One wave per token.
__global__ __launch_bounds__(64) void route_kernel(
        const float* __restrict__ z, long long z_stride, int E, int top, int groups, int keep,
        float weight_eps, int* __restrict__ chosen, float* __restrict__ weights) {
    extern __shared__ float re_lds[];            // s [E], group maxima [groups], allowed [groups]
    float* s = re_lds;
    float* gmax = s + E;
    int* allowed = (int*)(gmax + groups);
    const int lane = threadIdx.x, n = blockIdx.x;
    const float* zr = z + (size_t)n * z_stride;
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, zr[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
        const float p = expf(zr[e] - mx);
        s[e] = p;
        sum += p;
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < E; e += 64) s[e] *= inv;
    __syncthreads();
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
        float v = s[g * per];
        for (int i = 1; i < per; ++i) v = fmaxf(v, s[g * per + i]);
        gmax[g] = v;
    }
    __syncthreads();
    for (int g = lane; g < groups; g += 64) {
        int better = 0;
        for (int o = 0; o < groups; ++o)
            better += (gmax[o] > gmax[g] || (gmax[o] == gmax[g] && o < g)) ? 1 : 0;
        allowed[g] = better < keep;
    }
    __syncthreads();
    // the lane's experts that can still be chosen; -1 marks one that cannot
    float mine[RE_MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < RE_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        mine[i] = (e < E && allowed[e / per]) ? s[e] : -1.f;
    }
    float total = 0.f;
    float w_k = 0.f;                                    // lane k keeps the k-th choice
    int e_k = 0;
    for (int k = 0; k < top; ++k) {
        float best = -1.f;
        int at = E;
#pragma unroll
        for (int i = 0; i < RE_MAX_PER_LANE; ++i)
            if (mine[i] > best) {
                best = mine[i];
                at = lane + 64 * i;
            }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (ob > best || (ob == best && oa < at)) {
                best = ob;
                at = oa;
            }
        }
        if ((at & 63) == lane) {
#pragma unroll
            for (int i = 0; i < RE_MAX_PER_LANE; ++i)
                if (lane + 64 * i == at) mine[i] = -1.f;
        }
        total += best;
        if (lane == k) {
            w_k = best;
            e_k = at;
        }
    }
    const float norm = 1.f / (total + weight_eps);
    if (lane < top) {
        chosen[(size_t)n * top + lane] = e_k;
        weights[(size_t)n * top + lane] = w_k * norm;
    }
}

extern "C" int gfa_route(const float* z, long long z_stride, int n_tokens, int E, int top, int groups,
                         int keep, float weight_eps, int* chosen, float* weights,
                         hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (E <= 0 || E > 64 * RE_MAX_PER_LANE || groups <= 0 || E % groups || keep < 1 || keep > groups ||
            top < 1 || top > 64 || top > keep * (E / groups))
        return (int)hipErrorInvalidValue;
    const size_t shmem = sizeof(float) * (size_t)(E + 2 * groups);
    route_kernel<<<n_tokens, 64, shmem, stream>>>(z, z_stride, E, top, groups, keep, weight_eps,
                                                   chosen, weights);
    return GFA_LAUNCH_RESULT();
}

// 0 silu, 1 gelu (tanh form), 3 gelu (exact); the numbers of ops.kernels.ACTIVATIONS
__device__ __forceinline__ float re_activation(float z, int act) {
    if (act == 0) return z / (1.f + expf(-z));
    if (act == 1) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return 0.5f * z * (1.f + erff(z * 0.7071067811865476f));
}

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* f) {
        const uint4 raw = stream_load16(p);
        const uint32_t* w = (const uint32_t*)&raw;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <> struct Vec8<float> {
    static __device__ __forceinline__ void load(const float* p, float* f) {
        const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
        f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
};

// dot of a weight row with a vector in shared memory, over the lanes of a wave; every lane
// gets the sum.  The order of additions depends on K only.
template <typename T>
__device__ __forceinline__ float re_row_dot(const T* __restrict__ w, const float* __restrict__ x,
                                            int K, int lane) {
    float acc = 0.f;
    if (K % 8 == 0) {
        for (int k = lane * 8; k < K; k += 512) {
            float f[8];
            Vec8<T>::load(w + k, f);
#pragma unroll
            for (int t = 0; t < 8; ++t) acc = fmaf(f[t], x[k + t], acc);
        }
    } else {
        for (int k = lane; k < K; k += 64) acc = fmaf(load_as_float(w + k), x[k], acc);
    }
    return wave_sum(acc);
}

#define RE_THREADS 256
#define RE_ROWS 16                  // weight rows per workgroup: four per wave

// h[pair, f] = act(W_up[e(pair)][f, :] . x[token(pair), :]);  grid (F / RE_ROWS, pairs)
template <typename T>
__global__ __launch_bounds__(RE_THREADS) void expert_up_kernel(
        const T* __restrict__ x, const T* __restrict__ w_up, const int* __restrict__ chosen,
        T* __restrict__ h, int top, int D, int F, int act) {
    extern __shared__ float re_x[];
    const int pair = blockIdx.y, n = pair / top;
    const int e = chosen[pair];
    for (int d = threadIdx.x; d < D; d += RE_THREADS) re_x[d] = load_as_float(x + (size_t)n * D + d);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const T* w = w_up + (size_t)e * F * D;
    for (int r = wave; r < RE_ROWS; r += RE_THREADS / 64) {
        const int f = blockIdx.x * RE_ROWS + r;
        if (f >= F) break;
        const float v = re_row_dot<T>(w + (size_t)f * D, re_x, D, lane);
        if (lane == 0) store_from_float(h + (size_t)pair * F + f, re_activation(v, act));
    }
}

// y[n, c] (+)= sum_k weight[n, k] W_down[e_k][c, :] . h[n, k, :];  grid (D / RE_ROWS, tokens)
template <typename T>
__global__ __launch_bounds__(RE_THREADS) void expert_down_kernel(
        const T* __restrict__ h, const T* __restrict__ w_down, const int* __restrict__ chosen,
        const float* __restrict__ weights, float* __restrict__ y, int top, int D, int F,
        int accumulate) {
    extern __shared__ float re_h[];                    // [top][F]
    const int n = blockIdx.y;
    for (int i = threadIdx.x; i < top * F; i += RE_THREADS)
        re_h[i] = load_as_float(h + (size_t)n * top * F + i);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int r = wave; r < RE_ROWS; r += RE_THREADS / 64) {
        const int c = blockIdx.x * RE_ROWS + r;
        if (c >= D) break;
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = chosen[(size_t)n * top + k];
            const float v = re_row_dot<T>(w_down + ((size_t)e * D + c) * F, re_h + (size_t)k * F, F, lane);
            acc = fmaf(weights[(size_t)n * top + k], v, acc);
        }
        if (lane == 0) {
            float* o = y + (size_t)n * D + c;
            *o = accumulate ? *o + acc : acc;
        }
    }
}

extern "C" int gfa_experts_few_rows(const void* x, const void* w_up, const void* w_down,
                                    const int* chosen, const float* weights, void* h, float* y,
                                    int n_tokens, int top, int D, int F, int act, int accumulate,
                                    int is_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (top <= 0 || D <= 0 || F <= 0 || (act != 0 && act != 1 && act != 3) || n_tokens * (long long)top > 65535
            || n_tokens > 65535)
        return (int)hipErrorInvalidValue;
    const size_t up_lds = sizeof(float) * (size_t)D, down_lds = sizeof(float) * (size_t)top * F;
    if (up_lds > 64 * 1024 || down_lds > 64 * 1024) return (int)hipErrorInvalidValue;
    dim3 up_grid((F + RE_ROWS - 1) / RE_ROWS, n_tokens * top), down_grid((D + RE_ROWS - 1) / RE_ROWS, n_tokens);
    if (is_bf16) {
        expert_up_kernel<bf16_t><<<up_grid, RE_THREADS, up_lds, stream>>>(
            (const bf16_t*)x, (const bf16_t*)w_up, chosen, (bf16_t*)h, top, D, F, act);
        expert_down_kernel<bf16_t><<<down_grid, RE_THREADS, down_lds, stream>>>(
            (const bf16_t*)h, (const bf16_t*)w_down, chosen, weights, y, top, D, F, accumulate);
    } else {
        expert_up_kernel<float><<<up_grid, RE_THREADS, up_lds, stream>>>(
            (const float*)x, (const float*)w_up, chosen, (float*)h, top, D, F, act);
        expert_down_kernel<float><<<down_grid, RE_THREADS, down_lds, stream>>>(
            (const float*)h, (const float*)w_down, chosen, weights, y, top, D, F, accumulate);
    }
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// For steps of many rows the pairs are put in the order of their experts, so that each
// expert's rows are one product of the matrix library.  One workgroup: counts per expert,
// their running sum (offsets [E + 1]), and for every pair its place in that order
// (place[pair]; order[place] = pair).  The order of an expert's pairs among themselves is
// whatever the atomics give: each pair's row is computed by itself, so it does not matter.
__global__ __launch_bounds__(1024) void expert_order_kernel(
        const int* __restrict__ chosen, int n_pairs, int E, int* __restrict__ offsets,
        int* __restrict__ order, int* __restrict__ place) {
    extern __shared__ int eo_lds[];                    // start [E + 1], cursor [E]
    int* start = eo_lds;
    int* cursor = eo_lds + E + 1;
    for (int e = threadIdx.x; e <= E; e += blockDim.x) start[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&start[chosen[p] + 1], 1);
    __syncthreads();
    if (threadIdx.x == 0)
        for (int e = 0; e < E; ++e) start[e + 1] += start[e];
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) {
        offsets[e] = start[e];
        if (e < E) cursor[e] = start[e];
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int at = atomicAdd(&cursor[chosen[p]], 1);
        order[at] = p;
        place[p] = at;
    }
}

extern "C" int gfa_expert_order(const int* chosen, int n_pairs, int E, int* offsets, int* order,
                                int* place, hipStream_t stream) {
    if (n_pairs <= 0) return 0;
    if (E <= 0 || E > 8192) return (int)hipErrorInvalidValue;
    expert_order_kernel<<<1, 1024, sizeof(int) * (size_t)(2 * E + 1), stream>>>(chosen, n_pairs, E, offsets,
                                                                           order, place);
    return GFA_LAUNCH_RESULT();
}

// xs[i, :] = x[order[i] / top, :]: the tokens' rows in the order of their experts
template <typename T>
__global__ void gather_pairs_kernel(const T* __restrict__ x, const int* __restrict__ order,
                                    T* __restrict__ xs, int top, int D) {
    const T* src = x + (size_t)(order[blockIdx.x] / top) * D;
    T* dst = xs + (size_t)blockIdx.x * D;
    if (sizeof(T) == 2 && D % 8 == 0) {
        for (int d = threadIdx.x; d < D / 8; d += blockDim.x) ((uint4*)dst)[d] = ((const uint4*)src)[d];
    } else {
        for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = src[d];
    }
}

extern "C" int gfa_gather_pairs(const void* x, const int* order, void* xs, int n_pairs, int top, int D,
                                int is_bf16, hipStream_t stream) {
    if (n_pairs <= 0) return 0;
    if (is_bf16)
        gather_pairs_kernel<bf16_t><<<n_pairs, 256, 0, stream>>>((const bf16_t*)x, order, (bf16_t*)xs, top, D);
    else
        gather_pairs_kernel<float><<<n_pairs, 256, 0, stream>>>((const float*)x, order, (float*)xs, top, D);
    return GFA_LAUNCH_RESULT();
}

// y[n, :] (+)= sum_k weight[n, k] ys[place[n top + k], :], in the order of the choice
template <typename T>
__global__ void combine_pairs_kernel(const T* __restrict__ ys, const int* __restrict__ place,
                                     const float* __restrict__ weights, float* __restrict__ y,
                                     int top, int D, int accumulate) {
    const int n = blockIdx.x;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k)
            acc = fmaf(weights[(size_t)n * top + k],
                       load_as_float(ys + (size_t)place[(size_t)n * top + k] * D + d), acc);
        float* o = y + (size_t)n * D + d;
        *o = accumulate ? *o + acc : acc;
    }
}

extern "C" int gfa_combine_pairs(const void* ys, const int* place, const float* weights, float* y,
                                 int n_tokens, int top, int D, int accumulate, int is_bf16,
                                 hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (is_bf16)
        combine_pairs_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)ys, place, weights, y,
                                                                   top, D, accumulate);
    else
        combine_pairs_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)ys, place, weights, y,
                                                                  top, D, accumulate);
    return GFA_LAUNCH_RESULT();
}
