// A mixture of experts: the router's choice per token and the chosen experts' products.
//
// Router (float arithmetic): s = softmax(z) over all E experts, or sigmoid(z); the choice is
// made on s plus an optional correction per expert; the experts form `groups` equal groups of
// neighbours, a group's score is its largest choice score (or the sum of its few largest),
// only experts of the `keep` best groups can be chosen, and of those the `top` with the
// largest choice scores are; a chosen expert's weight is its s over the sum of the chosen s
// (+ weight_eps).  Ties go to the lower index.
//
// Products, one (token, chosen expert) pair at a time: h = act(W_up[e] x) - or, for gated
// experts whose W_up holds F gate rows and then F up rows, h = act(W_gate[e] x) * (W_up[e] x) - and
// y = sum_k weight_k W_down[e_k] h_k in the order of the choice.  Every output element is one
// chain of multiply-adds over its own inputs, so a token's result does not depend on what
// else the step holds.  These kernels serve the float32 engine and the steps of few rows;
// the weights of an expert are stacked: W_up [E, F, D], W_down [E, D, F].
#include "common.h"

#define RE_MAX_PER_LANE 16          // experts per lane of the router's wave: E <= 1024
#define RE_MAX_GROUP_TOP 8          // a group's score adds up at most this many of its scores

// One wave per token.  scoring 0: s = softmax(z) over all experts; 1: s = sigmoid(z), each
// expert by itself.  The CHOICE is made on c = s + correction (correction null: c = s): a
// group's score is the sum of its `group_top` largest c (1: its largest), the experts of the
// groups that are not kept count as minus infinity (c can be negative), and the `top`
// largest c are chosen; the WEIGHTS are the chosen experts' s over their sum.
__global__ __launch_bounds__(64) void route_kernel(
        const float* __restrict__ z, long long z_stride, int E, int top, int groups, int keep,
        float weight_eps, int scoring, const float* __restrict__ correction, int group_top,
        int* __restrict__ chosen, float* __restrict__ weights) {
    extern __shared__ float re_lds[];            // s [E], c [E], group scores [groups], allowed [groups]
    float* s = re_lds;
    float* c = s + E;
    float* gscore = c + E;
    int* allowed = (int*)(gscore + groups);
    const int lane = threadIdx.x, n = blockIdx.x;
    const float* zr = z + (size_t)n * z_stride;
    if (scoring == 0) {
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
    } else {
        for (int e = lane; e < E; e += 64) s[e] = 1.f / (1.f + expf(-zr[e]));
    }
    for (int e = lane; e < E; e += 64) c[e] = s[e] + (correction ? correction[e] : 0.f);
    __syncthreads();
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
        // the sum of the group's largest scores: the largest, then the largest of the rest, ...
        int taken[RE_MAX_GROUP_TOP];
        float total = 0.f;
        for (int t = 0; t < group_top && t < per; ++t) {
            float v = -INFINITY;
            int at = -1;
            for (int i = 0; i < per; ++i) {
                bool used = false;
                for (int u = 0; u < t; ++u) used = used || taken[u] == i;
                if (!used && (at < 0 || c[g * per + i] > v)) {
                    v = c[g * per + i];
                    at = i;
                }
            }
            taken[t] = at;
            total += v;
        }
        gscore[g] = total;
    }
    __syncthreads();
    for (int g = lane; g < groups; g += 64) {
        int better = 0;
        for (int o = 0; o < groups; ++o)
            better += (gscore[o] > gscore[g] || (gscore[o] == gscore[g] && o < g)) ? 1 : 0;
        allowed[g] = better < keep;
    }
    __syncthreads();
    // the lane's experts that can still be chosen; minus infinity marks one that cannot
    float mine[RE_MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < RE_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        mine[i] = (e < E && allowed[e / per]) ? c[e] : -INFINITY;
    }
    float total = 0.f;
    float w_k = 0.f;                                    // lane k keeps the k-th choice
    int e_k = 0;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
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
        if (at >= E) at = 0;                            // scores that are no number: any expert
        if ((at & 63) == lane) {
#pragma unroll
            for (int i = 0; i < RE_MAX_PER_LANE; ++i)
                if (lane + 64 * i == at) mine[i] = -INFINITY;
        }
        const float picked = s[at];
        total += picked;
        if (lane == k) {
            w_k = picked;
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
                         int keep, float weight_eps, int scoring, const float* correction,
                         int group_top, int* chosen, float* weights, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (E <= 0 || E > 64 * RE_MAX_PER_LANE || groups <= 0 || E % groups || keep < 1 || keep > groups ||
            top < 1 || top > 64 || top > keep * (E / groups) || (scoring != 0 && scoring != 1) ||
            group_top < 1 || group_top > RE_MAX_GROUP_TOP)
        return (int)hipErrorInvalidValue;
    const size_t shmem = sizeof(float) * (size_t)(2 * E + 2 * groups);
    route_kernel<<<n_tokens, 64, shmem, stream>>>(z, z_stride, E, top, groups, keep, weight_eps,
                                                   scoring, correction, group_top, chosen, weights);
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
        T* __restrict__ h, int top, int D, int F, int act, int gated) {
    extern __shared__ float re_x[];
    const int pair = blockIdx.y, n = pair / top;
    const int e = chosen[pair];
    for (int d = threadIdx.x; d < D; d += RE_THREADS) re_x[d] = load_as_float(x + (size_t)n * D + d);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const T* w = w_up + (size_t)e * (gated ? 2 : 1) * F * D;
    for (int r = wave; r < RE_ROWS; r += RE_THREADS / 64) {
        const int f = blockIdx.x * RE_ROWS + r;
        if (f >= F) break;
        float v = re_activation(re_row_dot<T>(w + (size_t)f * D, re_x, D, lane), act);
        if (gated) v *= re_row_dot<T>(w + (size_t)(F + f) * D, re_x, D, lane);
        if (lane == 0) store_from_float(h + (size_t)pair * F + f, v);
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
                                    int n_tokens, int top, int D, int F, int act, int gated,
                                    int accumulate, int is_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (top <= 0 || D <= 0 || F <= 0 || (act != 0 && act != 1 && act != 3) || n_tokens * (long long)top > 65535
            || n_tokens > 65535)
        return (int)hipErrorInvalidValue;
    const size_t up_lds = sizeof(float) * (size_t)D, down_lds = sizeof(float) * (size_t)top * F;
    if (up_lds > 64 * 1024 || down_lds > 64 * 1024) return (int)hipErrorInvalidValue;
    dim3 up_grid((F + RE_ROWS - 1) / RE_ROWS, n_tokens * top), down_grid((D + RE_ROWS - 1) / RE_ROWS, n_tokens);
    if (is_bf16) {
        expert_up_kernel<bf16_t><<<up_grid, RE_THREADS, up_lds, stream>>>(
            (const bf16_t*)x, (const bf16_t*)w_up, chosen, (bf16_t*)h, top, D, F, act, gated);
        expert_down_kernel<bf16_t><<<down_grid, RE_THREADS, down_lds, stream>>>(
            (const bf16_t*)h, (const bf16_t*)w_down, chosen, weights, y, top, D, F, accumulate);
    } else {
        expert_up_kernel<float><<<up_grid, RE_THREADS, up_lds, stream>>>(
            (const float*)x, (const float*)w_up, chosen, (float*)h, top, D, F, act, gated);
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

// The same rows with every expert's share padded to `cap` rows, for one batched product over
// all experts: xs[e, i, :] = x[order[offsets[e] + i] / top, :] for i < offsets[e + 1] - offsets[e],
// zero beyond.  Grid (cap, E).
template <typename T>
__global__ void gather_pairs_padded_kernel(const T* __restrict__ x, const int* __restrict__ order,
                                           const int* __restrict__ offsets, T* __restrict__ xs,
                                           int top, int D, int cap) {
    const int e = blockIdx.y, i = blockIdx.x;
    const int lo = offsets[e], count = offsets[e + 1] - lo;
    T* dst = xs + ((size_t)e * cap + i) * D;
    if (i >= count) {
        for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = (T)0;
        return;
    }
    const T* src = x + (size_t)(order[lo + i] / top) * D;
    if (sizeof(T) == 2 && D % 8 == 0) {
        for (int d = threadIdx.x; d < D / 8; d += blockDim.x) ((uint4*)dst)[d] = ((const uint4*)src)[d];
    } else {
        for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = src[d];
    }
}

extern "C" int gfa_gather_pairs_padded(const void* x, const int* order, const int* offsets, void* xs,
                                       int E, int cap, int top, int D, int is_bf16,
                                       hipStream_t stream) {
    if (E <= 0 || cap <= 0) return 0;
    if (E > 65535) return (int)hipErrorInvalidValue;
    dim3 grid(cap, E);
    if (is_bf16)
        gather_pairs_padded_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, order, offsets,
                                                                     (bf16_t*)xs, top, D, cap);
    else
        gather_pairs_padded_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, order, offsets,
                                                                    (float*)xs, top, D, cap);
    return GFA_LAUNCH_RESULT();
}

// padded[p] = chosen[p] * cap + place[p] - offsets[chosen[p]]: where pair p's row lies when every
// expert's share is padded to `cap` rows
__global__ void padded_places_kernel(const int* __restrict__ place, const int* __restrict__ chosen,
                                     const int* __restrict__ offsets, int* __restrict__ padded,
                                     int n_pairs, int cap) {
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_pairs) return;
    const int e = chosen[p];
    padded[p] = e * cap + place[p] - offsets[e];
}

extern "C" int gfa_padded_places(const int* place, const int* chosen, const int* offsets, int* padded,
                                 int n_pairs, int cap, hipStream_t stream) {
    if (n_pairs <= 0) return 0;
    padded_places_kernel<<<(n_pairs + 255) / 256, 256, 0, stream>>>(place, chosen, offsets, padded,
                                                                    n_pairs, cap);
    return GFA_LAUNCH_RESULT();
}

// y[n, :] (+)= sum_k weight[n, k] ys[place[n top + k], :], in the order of the choice
template <typename T>
__global__ void combine_pairs_kernel(const T* __restrict__ ys, const int* __restrict__ place,
                                     const float* __restrict__ weights, float* __restrict__ y,
                                     int top, int D, int accumulate) {
    const int n = blockIdx.x;
    for (int d = blockIdx.y * blockDim.x + threadIdx.x; d < D; d += gridDim.y * blockDim.x) {
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
    // few tokens: a row's elements are spread over several workgroups
    int parts = (D + 255) / 256;
    if (parts > 32) parts = 32;
    if (n_tokens >= 1024) parts = 1;
    dim3 grid(n_tokens, parts);
    if (is_bf16)
        combine_pairs_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)ys, place, weights, y,
                                                               top, D, accumulate);
    else
        combine_pairs_kernel<float><<<grid, 256, 0, stream>>>((const float*)ys, place, weights, y,
                                                              top, D, accumulate);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Single-token steps in bfloat16: the pairs in the order of their experts (expert_order_kernel,
// nothing is read on the host), and per expert ONE pass over its matrix for all of its rows.
//
//   out[offsets[e] + i, n] = f(W[e][n, :] . x[row(offsets[e] + i), :]),  i < offsets[e + 1] - offsets[e]
//   row(p) = order[p] / top if order is given (the token of the pair at place p), else p.
//
// Grid (column tiles, experts).  A workgroup of an expert without rows ends at once; the others
// walk K in pieces of 128: the expert's rows of x (up to CT * 16 at a time, gathered) go once
// per workgroup into LDS, double-buffered; each wave streams 16 rows of W through a padded LDS
// tile of its own into the operand layout of v_mfma_f32_16x16x32_bf16, DEPTH pieces ahead.  XD (up to
// 16 rows, for steps of very few tokens, where few experts have rows at all and the chip is not
// full): no shared x and no barriers while K is walked; a lane reads its own operand pieces of
// x from memory, four pieces ahead like W; the workgroup's four waves take the same 16 columns
// and a quarter of K each, and the first adds their sums in the waves' order (four times the
// workgroups).  A
// row of x meets only its own lanes of the operand and K is walked in the same order whatever
// the step holds, so a pair's result does not depend on the other pairs.  act < 0: the float
// sums are stored; else act(sum) as bfloat16.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 re_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float re_floatx4_t;
union ReFrag {
    uint4 u;
    re_bf16x8_t v;
};

#define GR_SUBK 128
#define GR_PITCH (GR_SUBK * 2 + 16)           // bytes per staged row: 256 + pad against conflicts
#define GR_TILE (16 * GR_PITCH)
#define GR_NW 4                               // waves per workgroup: 64 columns

template <int CT, int DEPTH, bool XD>
__global__ __launch_bounds__(GR_NW * 64) void grouped_rows_kernel(
        const bf16_t* __restrict__ x, const int* __restrict__ order, int top,
        const bf16_t* __restrict__ w, const int* __restrict__ offsets, void* __restrict__ out,
        int N, int K, int act) {
    constexpr int NT = GR_NW * 64;
    constexpr int XBYTES = CT * 16 * GR_PITCH;
    constexpr int XPER = CT;                               // CT * 16 rows of 16 pieces over 256 threads
    extern __shared__ __attribute__((aligned(16))) char gr_smem[];
    const int e = blockIdx.y;
    const int lo = offsets[e], hi = offsets[e + 1];
    if (hi <= lo) return;                                  // the same for every thread of the workgroup
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fi = lane & 15, fg = lane >> 4;
    const int lrow = lane >> 4, lchunk = lane & 15;
    char* stage = gr_smem + (XD ? 0 : 2 * XBYTES) + wave * GR_TILE;
    const int n0w = XD ? blockIdx.x * 16 : (blockIdx.x * GR_NW + wave) * 16;
    const int T = (K + GR_SUBK - 1) / GR_SUBK;
    const bf16_t* we = w + (size_t)e * N * K;
    const bf16_t* wsrc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int n = n0w + lrow + 4 * j;
        if (n >= N) n = N - 1;                             // read again, never stored
        wsrc[j] = we + (size_t)n * K + lchunk * 8;
    }

    for (int m0 = lo; m0 < hi; m0 += CT * 16) {
        const int M = (hi - m0 < CT * 16) ? hi - m0 : CT * 16;
        const bf16_t* xsrc[XPER];
#pragma unroll
        for (int i = 0; i < XPER; ++i) {
            const int c = threadIdx.x + i * NT;
            const int row = c >> 4, chunk = c & 15;
            if (row < M) {
                const int src = order ? order[m0 + row] / top : m0 + row;
                xsrc[i] = x + (size_t)src * K + chunk * 8;
            } else {
                xsrc[i] = nullptr;
            }
        }
        re_floatx4_t acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[ct] = re_floatx4_t{0.f, 0.f, 0.f, 0.f};
        uint4 wr[DEPTH][4], xr[XPER];
        // XD: the lane's own operand pieces of x straight from memory (row fi, k group fg)
        uint4 xd[XD ? DEPTH : 1][4];
        const bf16_t* xrow = nullptr;
        if (XD && fi < M) xrow = x + (size_t)(order ? order[m0 + fi] / top : m0 + fi) * K + fg * 8;
        auto load_xd = [&](int t, uint4 (&regs)[4]) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bool ok = xrow != nullptr && t * GR_SUBK + s * 32 + fg * 8 < K;
                regs[s] = ok ? *(const uint4*)(xrow + (size_t)t * GR_SUBK + s * 32) : make_uint4(0, 0, 0, 0);
            }
        };
        auto load_w = [&](int t, uint4 (&regs)[4]) {
            const bool ok = t * GR_SUBK + lchunk * 8 < K;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                regs[j] = ok ? stream_load16(wsrc[j] + (size_t)t * GR_SUBK) : make_uint4(0, 0, 0, 0);
        };
        auto stage_w = [&](uint4 (&regs)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *(uint4*)(stage + (lrow + 4 * j) * GR_PITCH + lchunk * 16) = regs[j];
        };
        auto load_x = [&](int t) {
#pragma unroll
            for (int i = 0; i < XPER; ++i) {
                const int c = threadIdx.x + i * NT;
                const bool ok = xsrc[i] != nullptr && t * GR_SUBK + (c & 15) * 8 < K;
                xr[i] = ok ? *(const uint4*)(xsrc[i] + (size_t)t * GR_SUBK) : make_uint4(0, 0, 0, 0);
            }
        };
        auto store_x = [&](int buf) {
#pragma unroll
            for (int i = 0; i < XPER; ++i) {
                const int c = threadIdx.x + i * NT;
                *(uint4*)(gr_smem + buf * XBYTES + (c >> 4) * GR_PITCH + (c & 15) * 16) = xr[i];
            }
        };
        auto multiply = [&](int buf) {
            const char* xb = gr_smem + buf * XBYTES;
#pragma unroll
            for (int s = 0; s < GR_SUBK / 32; ++s) {
                ReFrag a;
                a.u = *(const uint4*)(stage + fi * GR_PITCH + (s * 4 + fg) * 16);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    if (ct * 16 >= M) break;               // no rows in this tile (M is the workgroup's)
                    ReFrag b;
                    b.u = *(const uint4*)(xb + (ct * 16 + fi) * GR_PITCH + (s * 4 + fg) * 16);
                    acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[ct], 0, 0, 0);
                }
            }
        };

        if (XD) {
            // no shared x, no barriers while K is walked: the workgroup's waves take the same 16
            // columns and a quarter of K each; their sums are added in the waves' order
            const int per_wave = (T + GR_NW - 1) / GR_NW;
            const int t_lo = wave * per_wave;
            const int t_hi = (t_lo + per_wave < T) ? t_lo + per_wave : T;
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
                if (t_lo + u < t_hi) {
                    load_w(t_lo + u, wr[u]);
                    load_xd(t_lo + u, xd[XD ? u : 0]);
                }
            for (int t = t_lo; t < t_hi; t += DEPTH) {
#pragma unroll
                for (int u = 0; u < DEPTH; ++u) {
                    const int tt = t + u;
                    if (tt >= t_hi) break;
                    stage_w(wr[u]);
                    ReFrag b[4];
#pragma unroll
                    for (int s = 0; s < 4; ++s) b[s].u = xd[XD ? u : 0][s];
                    if (tt + DEPTH < t_hi) {
                        load_w(tt + DEPTH, wr[u]);
                        load_xd(tt + DEPTH, xd[XD ? u : 0]);
                    }
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        ReFrag a;
                        a.u = *(const uint4*)(stage + fi * GR_PITCH + (s * 4 + fg) * 16);
                        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b[s].v, acc[0], 0, 0, 0);
                    }
                }
            }
            float* red = (float*)(gr_smem + GR_NW * GR_TILE);          // [waves][64 lanes][4]
#pragma unroll
            for (int j = 0; j < 4; ++j) red[(wave * 64 + lane) * 4 + j] = acc[0][j];
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float v = red[lane * 4 + j];
                    for (int o = 1; o < GR_NW; ++o) v += red[(o * 64 + lane) * 4 + j];
                    acc[0][j] = v;
                }
            }
            __syncthreads();                               // before the next chunk's sums
        } else {
        __syncthreads();                                   // the chunk before has been multiplied
        load_x(0);
#pragma unroll
        for (int u = 0; u < DEPTH; ++u)
            if (u < T) load_w(u, wr[u]);
        store_x(0);
        __syncthreads();
        // piece t: x in buffer t & 1, W in wr[t % DEPTH], asked for DEPTH pieces ahead
        for (int t = 0; t < T; t += DEPTH) {
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                const int tt = t + u;
                if (tt >= T) break;
                if (tt + 1 < T) load_x(tt + 1);
                stage_w(wr[u]);
                if (tt + DEPTH < T) load_w(tt + DEPTH, wr[u]);
                multiply(u & 1);
                if (tt + 1 < T) store_x((u + 1) & 1);
                __syncthreads();
            }
        }
        }

        // lane: columns n0w + 4 fg .. + 3 of the result, row ct * 16 + fi of the chunk
        if (n0w < N && (!XD || wave == 0)) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const int m = ct * 16 + fi;
                if (m >= M) continue;
                const int n = n0w + fg * 4;
                const size_t at = (size_t)(m0 + m) * N + n;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (n + j >= N) break;
                    const float v = acc[ct][j];
                    if (act < 0) ((float*)out)[at + j] = v;
                    else ((bf16_t*)out)[at + j] = float_to_bf16(re_activation(v, act));
                }
            }
        }
    }
}

// out [pairs, N] from x (rows by order / top, or by place) and W [E, N, K]; rows_at_most: the
// most rows one expert can have (the step's tokens), which sizes the tiles of x.
extern "C" int gfa_grouped_rows(const void* x, const int* order, int top, const void* w,
                                const int* offsets, void* out, int E, int N, int K, int act,
                                int rows_at_most, int x_direct, hipStream_t stream) {
    if (E <= 0 || N <= 0 || K <= 0 || K % 8 || top <= 0 || E > 65535) return (int)hipErrorInvalidValue;
    if (act >= 0 && act != 0 && act != 1 && act != 3) return (int)hipErrorInvalidValue;
    dim3 grid((N + GR_NW * 16 - 1) / (GR_NW * 16), E);
    dim3 grid_direct((N + 15) / 16, E);
#define GFA_LAUNCH_GROUPED(CTV, DV, XDV)                                                          \
    grouped_rows_kernel<CTV, DV, XDV><<<(XDV ? grid_direct : grid), GR_NW * 64,                   \
        (XDV ? GR_NW * 64 * 4 * sizeof(float) : 2 * CTV * 16 * GR_PITCH) + GR_NW * GR_TILE, stream>>>( \
        (const bf16_t*)x, order, top, (const bf16_t*)w, offsets, out, N, K, act)
    if (rows_at_most <= 16 && x_direct) GFA_LAUNCH_GROUPED(1, 4, true);
    else if (rows_at_most <= 16) GFA_LAUNCH_GROUPED(1, 2, false);
    else if (rows_at_most <= 32) GFA_LAUNCH_GROUPED(2, 2, false);
    else GFA_LAUNCH_GROUPED(4, 2, false);
#undef GFA_LAUNCH_GROUPED
    return GFA_LAUNCH_RESULT();
}
