// Linear attention with a fixed decay per head (lightning attention): per sequence and head a
// float state S [dk, dv], zero at the sequence's start and kept in the cache's state slots:
//     q = silu(q'), k = silu(k'), v = silu(v')        (q', k', v': the projection's float sums;
//                                                      or q', k', v' themselves: `act` 0)
//     S' = decay_h S + k v^T          o = S'^T q
// Everything here is float arithmetic.  One slot's state: S [H][dk][dv].
//
// Two kernels: token by token (single-token steps and short runs), and a chunk of tokens at a
// time (prompts).  Inside a chunk that starts from S0, with a = decay_h and tokens t = 0, 1, ...:
//     o_t = a^(t+1) S0^T q_t + sum_{s<=t} a^(t-s) (k_s . q_t) v_s
//     S_L = a^L S0 + sum_s a^(L-1-s) k_s v_s^T
// which is the recurrence written out; every power of a has a non-negative exponent.
#include "common.h"

#define DM_THREADS 256
#define DM_COLS 32                      // columns of S (elements of v) per workgroup
#define DM_GROUPS (DM_THREADS / DM_COLS)

struct DMShape {
    int H, dk, dv;
    int row_width;                      // floats per row of proj
    int q_off, k_off, v_off;            // column offsets in a row of proj
    int act;                            // 1: q, k, v are silu of the row's values; 0: the values themselves
};

__device__ __forceinline__ float dm_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float dm_act(float z, int act) { return act ? dm_silu(z) : z; }

// Token by token.  grid (dv / DM_COLS, H, sequences).  Thread (c, g) = (tid % 32, tid / 32)
// holds rows g, g + 8, ... of column c of S in registers.
template <int RPT>
__global__ __launch_bounds__(DM_THREADS) void decayed_memory_scan_kernel(
        const float* __restrict__ proj, const float* __restrict__ decay, float* __restrict__ state,
        size_t slot_stride, const int* __restrict__ q_start, const int* __restrict__ slots,
        float* __restrict__ out, DMShape s) {
    __shared__ float qs[RPT * DM_GROUPS], ks[RPT * DM_GROUPS];
    __shared__ float red[DM_GROUPS][DM_COLS];
    const int tid = threadIdx.x, c = tid % DM_COLS, g = tid / DM_COLS;
    const int col = blockIdx.x * DM_COLS + c;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const S = state + (size_t)slots[b] * slot_stride + (size_t)h * s.dk * s.dv;
    const bool col_ok = col < s.dv;
    const float a = decay[h];

    float Sreg[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * DM_GROUPS;
        Sreg[r] = (col_ok && row < s.dk) ? S[(size_t)row * s.dv + col] : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        const float* row = proj + (size_t)t * s.row_width;
        for (int e = tid; e < RPT * DM_GROUPS; e += DM_THREADS) {
            qs[e] = e < s.dk ? dm_act(row[s.q_off + h * s.dk + e], s.act) : 0.f;
            ks[e] = e < s.dk ? dm_act(row[s.k_off + h * s.dk + e], s.act) : 0.f;
        }
        const float v = col_ok ? dm_act(row[s.v_off + h * s.dv + col], s.act) : 0.f;
        __syncthreads();
        float part = 0.f;
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            const int e = g + r * DM_GROUPS;
            Sreg[r] = fmaf(a, Sreg[r], ks[e] * v);
            part = fmaf(Sreg[r], qs[e], part);
        }
        red[g][c] = part;
        __syncthreads();
        if (g == 0 && col_ok) {
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < DM_GROUPS; ++r) o += red[r][c];
            out[(size_t)t * s.H * s.dv + (size_t)h * s.dv + col] = o;
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * DM_GROUPS;
        if (col_ok && row < s.dk) S[(size_t)row * s.dv + col] = Sreg[r];
    }
}

extern "C" int gfa_decayed_memory_scan(const float* proj, const float* decay, float* state,
                                       size_t slot_stride, const int* q_start, const int* slots,
                                       float* out, int n_seqs, int H, int dk, int dv, int row_width,
                                       int q_off, int k_off, int v_off, int act, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (dk > 64 * DM_GROUPS || H > 65535 || n_seqs > 65535) return (int)hipErrorInvalidValue;
    DMShape s{H, dk, dv, row_width, q_off, k_off, v_off, act};
    dim3 grid((dv + DM_COLS - 1) / DM_COLS, H, n_seqs);
    const int rpt = (dk + DM_GROUPS - 1) / DM_GROUPS;
#define DM_LAUNCH(R) decayed_memory_scan_kernel<R><<<grid, DM_THREADS, 0, stream>>>( \
        proj, decay, state, slot_stride, q_start, slots, out, s)
    if (rpt <= 4) DM_LAUNCH(4);
    else if (rpt <= 8) DM_LAUNCH(8);
    else if (rpt <= 16) DM_LAUNCH(16);
    else if (rpt <= 32) DM_LAUNCH(32);
    else DM_LAUNCH(64);
#undef DM_LAUNCH
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The same cell for runs of many tokens, a chunk of DC_L (32 or 64) tokens at a time.  With
// a = decay_h, S0 the state at the chunk's start and t, s = 0, 1, ... the chunk's tokens:
//     P[t][s] = (q_t . k_s) a^(t-s)  for s <= t
//     o_t = a^(t+1) (S0^T q_t) + sum_s P[t][s] v_s
//     S_L = a^L S0 + sum_s a^(L-1-s) k_s v_s^T
// The four products (scores, Q S0, P V, the state's update) run on the matrix cores in float
// (v_mfma_f32_16x16x4_f32: lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16] and holds
// C[4 (l / 16) .. +3][l % 16]).  grid (dv / DC_COLS, H, sequences), eight threads per token of a
// chunk; q, k, v of the chunk, the weighted scores and the workgroup's columns of S are in
// shared memory; a chunk's rows are fetched a chunk ahead.
#define DC_COLS 32

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float dc_floatx4_t;

// rows of q and k in shared memory: dk filled up to a multiple of 16 (the matrix cores' tiles)
// plus four floats, so that the sixteen rows a load touches lie in different banks
__host__ __device__ inline int dc_padded(int dk) { return (dk + 15) / 16 * 16; }
__host__ __device__ inline int dc_row_stride(int dk) { return dc_padded(dk) + 4; }

__device__ __forceinline__ float4 dm_act4(float4 x, int act) {
    return act ? make_float4(dm_silu(x.x), dm_silu(x.y), dm_silu(x.z), dm_silu(x.w)) : x;
}

template <int DC_L>
__global__ __launch_bounds__(DC_L * 8) void decayed_memory_chunk_kernel(
        const float* __restrict__ proj, const float* __restrict__ decay, float* __restrict__ state,
        size_t slot_stride, const int* __restrict__ q_start, const int* __restrict__ slots,
        float* __restrict__ out, DMShape s) {
    extern __shared__ __attribute__((aligned(16))) float dc_lds[];
    constexpr int NT = DC_L * 8;                 // threads: eight per token of a chunk
    constexpr int NWV = NT / 64;                 // waves
    constexpr int DC_PS = DC_L + 1;
    const int KS = dc_row_stride(s.dk);
    const int dkp = dc_padded(s.dk);
    float* Qs = dc_lds;                          // [DC_L][KS]
    float* Ks = Qs + DC_L * KS;                  // [DC_L][KS]
    float* Vs = Ks + DC_L * KS;                  // [DC_L][DC_COLS]
    float* Ps = Vs + DC_L * DC_COLS;             // [DC_L][DC_PS]
    float* Ss = Ps + DC_L * DC_PS;               // [dkp][DC_COLS]
    float* pw = Ss + dkp * DC_COLS;              // [DC_L + 1] a^i
    float* ws = pw + DC_L + 1;                   // [DC_L] a^(L - 1 - s), 0 beyond the chunk's end
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col0 = blockIdx.x * DC_COLS;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const S = state + (size_t)slots[b] * slot_stride + (size_t)h * s.dk * s.dv;

    for (int e = tid; e < dkp * DC_COLS; e += NT) {
        const int d = e / DC_COLS, c = e % DC_COLS;
        Ss[e] = (d < s.dk && col0 + c < s.dv) ? S[(size_t)d * s.dv + col0 + c] : 0.f;
    }
    for (int e = tid; e < 2 * DC_L * KS; e += NT) Qs[e] = 0.f;      // q and k: the filling stays zero
    if (tid == 0) {
        // by repeated multiplication, as the token-by-token kernel decays its state
        const float a = decay[h];
        float p = 1.f;
        for (int i = 0; i <= DC_L; ++i) {
            pw[i] = p;
            p *= a;
        }
    }

    const int kq4 = s.dk / 4;
    const bool vec = s.dk % 4 == 0 && s.dv % 4 == 0 && s.row_width % 4 == 0 && s.q_off % 4 == 0
                     && s.k_off % 4 == 0 && s.v_off % 4 == 0 && s.dk <= 128;
    float4 rq[4], rk[4], rv;
    auto fetch = [&](int c0) {
        const int Lc = t1 - c0 < DC_L ? t1 - c0 : DC_L;
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + NT * i, t = e / kq4, d4 = e - t * kq4;
            rq[i] = rk[i] = zero;
            if (t < Lc) {
                const float* row = proj + (size_t)(c0 + t) * s.row_width + h * s.dk + d4 * 4;
                rq[i] = *(const float4*)(row + s.q_off);
                rk[i] = *(const float4*)(row + s.k_off);
            }
        }
        {
            const int t = tid >> 3, c4 = (tid & 7) * 4;
            rv = zero;
            if (t < Lc && col0 + c4 < s.dv)
                rv = *(const float4*)(proj + (size_t)(c0 + t) * s.row_width + s.v_off + h * s.dv + col0 + c4);
        }
    };
    if (vec && t0 < t1) fetch(t0);

    for (int c0 = t0; c0 < t1; c0 += DC_L) {
        const int Lc = t1 - c0 < DC_L ? t1 - c0 : DC_L;
        __syncthreads();                         // the chunk before is done with Qs .. Ss
        if (vec) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int e = tid + NT * i, t = e / kq4, d4 = e - t * kq4;
                if (t < DC_L) {
                    // silu(0) = 0: rows beyond the chunk's end stay zero
                    *(float4*)(Qs + t * KS + d4 * 4) = dm_act4(rq[i], s.act);
                    *(float4*)(Ks + t * KS + d4 * 4) = dm_act4(rk[i], s.act);
                }
            }
            *(float4*)(Vs + (tid >> 3) * DC_COLS + (tid & 7) * 4) = dm_act4(rv, s.act);
            if (c0 + DC_L < t1) fetch(c0 + DC_L);
        } else {
            for (int e = tid; e < DC_L * KS; e += NT) {
                const int t = e / KS, d = e - t * KS;
                const bool ok = t < Lc && d < s.dk;
                const float* row = proj + (size_t)(c0 + t) * s.row_width;
                Qs[e] = ok ? dm_act(row[s.q_off + h * s.dk + d], s.act) : 0.f;
                Ks[e] = ok ? dm_act(row[s.k_off + h * s.dk + d], s.act) : 0.f;
            }
            for (int e = tid; e < DC_L * DC_COLS; e += NT) {
                const int t = e / DC_COLS, c = e % DC_COLS;
                Vs[e] = (t < Lc && col0 + c < s.dv)
                    ? dm_act(proj[(size_t)(c0 + t) * s.row_width + s.v_off + h * s.dv + col0 + c], s.act) : 0.f;
            }
        }
        if (tid < DC_L) ws[tid] = tid < Lc ? pw[Lc - 1 - tid] : 0.f;
        __syncthreads();
        const int li = lane & 15, lg = lane >> 4;
        // scores of the chunk, decayed: the 16 x 16 tiles on and below the diagonal, handed out
        // over the waves
        for (int idx = wave; idx < (DC_L / 16) * (DC_L / 16 + 1) / 2; idx += NWV) {
            int ti = 0;
            while ((ti + 1) * (ti + 2) / 2 <= idx) ++ti;
            const int si = idx - ti * (ti + 1) / 2;
            dc_floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
            const float* qa = Qs + (ti * 16 + li) * KS + lg;
            const float* kb = Ks + (si * 16 + li) * KS + lg;
#pragma unroll 4
            for (int d0 = 0; d0 < dkp; d0 += 4)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[d0], kb[d0], acc, 0, 0, 0);
            const int ss = si * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = ti * 16 + lg * 4 + r;
                Ps[t * DC_PS + ss] = ss <= t ? acc[r] * pw[t - ss] : 0.f;
            }
        }
        __syncthreads();
        // o_t for the workgroup's columns: a^(t+1) (Q S0) + P V
        dc_floatx4_t num = {0.f, 0.f, 0.f, 0.f};
        const int oti = wave >> 1, oci = wave & 1;
        {
            const float* qa = Qs + (oti * 16 + li) * KS + lg;
            const float* sb = Ss + lg * DC_COLS + oci * 16 + li;
#pragma unroll 4
            for (int d0 = 0; d0 < dkp; d0 += 4)
                num = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[d0], sb[d0 * DC_COLS], num, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) num[r] *= pw[oti * 16 + lg * 4 + r + 1];
            const float* pa = Ps + (oti * 16 + li) * DC_PS + lg;
            const float* vb = Vs + lg * DC_COLS + oci * 16 + li;
#pragma unroll 4
            for (int s0 = 0; s0 < (oti + 1) * 16; s0 += 4)
                num = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[s0], vb[s0 * DC_COLS], num, 0, 0, 0);
        }
        __syncthreads();                         // Ss has been read by every wave
        {
            const int c = col0 + oci * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = oti * 16 + lg * 4 + r;
                if (t < Lc && c < s.dv)
                    out[(size_t)(c0 + t) * s.H * s.dv + (size_t)h * s.dv + c] = num[r];
            }
        }
        // the state after the chunk's last token: S = a^L S + (w K)^T V, a wave's tiles of 16
        // rows of S by 16 columns in turn
        {
            const float aL = pw[Lc];
            for (int tile = wave; tile < (dkp / 16) * 2; tile += NWV) {
                const int di = tile >> 1, ci = tile & 1;
                float* sc = Ss + (di * 16 + lg * 4) * DC_COLS + ci * 16 + li;
                dc_floatx4_t acc;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = aL * sc[r * DC_COLS];
                const float* ka = Ks + lg * KS + di * 16 + li;
                const float* vb = Vs + lg * DC_COLS + ci * 16 + li;
#pragma unroll
                for (int s0 = 0; s0 < DC_L; s0 += 4)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ws[s0 + lg] * ka[s0 * KS], vb[s0 * DC_COLS],
                                                              acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) sc[r * DC_COLS] = acc[r];
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < s.dk * DC_COLS; e += NT) {
        const int d = e / DC_COLS, c = e % DC_COLS;
        if (col0 + c < s.dv) S[(size_t)d * s.dv + col0 + c] = Ss[e];
    }
}

static int dc_lds_bytes(int dk, int L) {
    const int dkp = dc_padded(dk);
    return (int)sizeof(float) * (2 * L * dc_row_stride(dk) + L * DC_COLS + L * (L + 1)
                                 + dkp * DC_COLS + 2 * L + 1);
}

static int dc_lds_limit() {
    static int limit = -1;
    if (limit < 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess)
            v = 64 * 1024;
        limit = v;
    }
    return limit;
}

// 1 if the chunked kernel takes these sizes on this device
extern "C" int gfa_decayed_memory_chunks_take(int dk, int dv) {
    return dk >= 1 && dv >= 1 && dc_lds_bytes(dk, 32) <= 64 * 1024 ? 1 : 0;
}

// Chunks of 64 tokens (512 threads) where the device lets a workgroup have the shared memory
// for them, else chunks of 32 (256 threads, at most 64 KB): a longer chunk spreads the chain of
// barriers and the state's products over twice the tokens.
extern "C" int gfa_decayed_memory_chunks(const float* proj, const float* decay, float* state,
                                         size_t slot_stride, const int* q_start, const int* slots,
                                         float* out, int n_seqs, int H, int dk, int dv,
                                         int row_width, int q_off, int k_off, int v_off, int act,
                                         hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (H > 65535 || n_seqs > 65535) return (int)hipErrorInvalidValue;
    DMShape s{H, dk, dv, row_width, q_off, k_off, v_off, act};
    dim3 grid((dv + DC_COLS - 1) / DC_COLS, H, n_seqs);
    const int big = dc_lds_bytes(dk, 64);
    if (big <= dc_lds_limit() && big <= 160 * 1024) {
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute((const void*)decayed_memory_chunk_kernel<64>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
        decayed_memory_chunk_kernel<64><<<grid, 512, big, stream>>>(proj, decay, state, slot_stride,
                                                                   q_start, slots, out, s);
        return GFA_LAUNCH_RESULT();
    }
    const int small = dc_lds_bytes(dk, 32);
    if (small > 64 * 1024) return (int)hipErrorInvalidValue;
    decayed_memory_chunk_kernel<32><<<grid, 256, small, stream>>>(proj, decay, state, slot_stride,
                                                                 q_start, slots, out, s);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The heads' results side by side, normed in `groups` equal parts of a row (1: the whole row;
// H: every head by itself), times a weight per element (weight_width elements, used again and
// again along the row: the row's width for a weight per element, a head's size for one weight
// shared by the heads; null: no weight), times a gate of the gate projection (gate_act 0:
// sigmoid(g), 1: silu(g) = g sigmoid(g)); rounded once, to the type of the output
// projection's operand.
//     y[t, :] = o[t, :] * rsqrt(mean_over_part(o[t, :]^2) + eps) * weight[:] * gate(g[t, :])
// The gate's pre-activations lie in proj at column g_off.  One workgroup per token, the waves
// take the parts in turn.
template <typename T>
__global__ __launch_bounds__(1024) void row_norm_gate_kernel(
        const float* __restrict__ o, const float* __restrict__ weight, int weight_width,
        const float* __restrict__ proj, int row_width, int g_off, T* __restrict__ y, int width,
        int groups, int gate_act, float eps) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    const float* src = o + t * width;
    const float* gate = proj + t * row_width + g_off;
    if (groups == 1) {
        float ss = 0.f;
        for (int d = threadIdx.x; d < width; d += blockDim.x) ss = fmaf(src[d], src[d], ss);
        const float r = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
        for (int d = threadIdx.x; d < width; d += blockDim.x) {
            const float g = gate[d], sg = 1.f / (1.f + expf(-g));
            store_from_float(y + t * width + d, src[d] * r * (weight ? weight[d % weight_width] : 1.f)
                                                * (gate_act ? g * sg : sg));
        }
        return;
    }
    const int part = width / groups, lane = threadIdx.x & 63;
    for (int p = threadIdx.x >> 6; p < groups; p += blockDim.x >> 6) {
        const int base = p * part;
        float ss = 0.f;
        for (int d = lane; d < part; d += 64) ss = fmaf(src[base + d], src[base + d], ss);
        const float r = rsqrtf(wave_sum(ss) / (float)part + eps);
        for (int d = base + lane; d < base + part; d += 64) {
            const float g = gate[d], sg = 1.f / (1.f + expf(-g));
            store_from_float(y + t * width + d, src[d] * r * (weight ? weight[d % weight_width] : 1.f)
                                                * (gate_act ? g * sg : sg));
        }
    }
}

extern "C" int gfa_row_norm_gate(const float* o, const float* weight, int weight_width,
                                 const float* proj, int row_width, int g_off, void* y, int y_bf16,
                                 int n_tokens, int width, int groups, int gate_act, float eps,
                                 hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (groups < 1 || width % groups || (weight && (weight_width < 1 || width % weight_width)))
        return (int)hipErrorInvalidValue;
    const int threads = width > 1024 ? 1024 : 256;       // an element or a few per thread
    if (y_bf16)
        row_norm_gate_kernel<bf16_t><<<n_tokens, threads, 0, stream>>>(
            o, weight, weight_width, proj, row_width, g_off, (bf16_t*)y, width, groups, gate_act, eps);
    else
        row_norm_gate_kernel<float><<<n_tokens, threads, 0, stream>>>(
            o, weight, weight_width, proj, row_width, g_off, (float*)y, width, groups, gate_act, eps);
    return GFA_LAUNCH_RESULT();
}
