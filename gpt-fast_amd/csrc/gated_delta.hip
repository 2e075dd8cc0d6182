// The gated delta rule behind short causal convolutions: per sequence and head a float state
// S [dk, dv], zero at the sequence's start and kept in the cache's state slots, and the last
// taps - 1 inputs of every convolved channel.
//
//     q', k', v' = the projection's float sums; each channel passes a causal convolution over
//     time (taps [C, K], the last column weighs the current token, zeros before the start)
//     and then silu
//     q = q' / sqrt(sum(q'^2) + unit_eps) * q_scale      k = k' / sqrt(sum(k'^2) + unit_eps)
//     beta = sigmoid(b')      g = exp(-exp(A_log_h) softplus(a' + dt_bias_h))
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
//
// Head h of v, beta, g and o uses head h / (H / G) of q and k.  Everything here is float
// arithmetic.  One slot's state: S [H][dk][dv], then the convolutions' tails [K - 1][C], oldest
// first, C = 2 G dk + H dv channels in the order q, k, v.
#include "common.h"

#define GD_THREADS 256
#define GD_COLS 32                      // columns of S (elements of v) per workgroup
#define GD_GROUPS (GD_THREADS / GD_COLS)
#define GD_MAX_TAPS 16

__device__ __forceinline__ float gd_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float gd_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// y[n, c] = silu(sum_j taps[c, j] x[n - (K - 1) + j, c]) over the tokens of n's own sequence;
// inputs before the step come from the sequence's tail, which is left as it is.  The
// convolved channels are the first C columns of a row of proj.  One thread per (token, channel).
__global__ __launch_bounds__(256) void short_conv_kernel(
        const float* __restrict__ proj, int row_width, const float* __restrict__ taps, int K, int C,
        const float* __restrict__ state, size_t slot_stride, size_t tail_off,
        const int* __restrict__ tok_seq, const int* __restrict__ q_start,
        const int* __restrict__ slots, float* __restrict__ y, int n_tokens) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)n_tokens * C) return;
    const int n = (int)(idx / C), c = (int)(idx - (long long)n * C);
    const int b = tok_seq[n];
    const int first = q_start[b];
    const float* tail = state + (size_t)slots[b] * slot_stride + tail_off;
    float acc = 0.f;
    for (int j = 0; j < K; ++j) {
        const int src = n - (K - 1) + j;               // a row of this step, if it is the sequence's
        const float x = src >= first ? proj[(size_t)src * row_width + c]
                                     : tail[(size_t)(K - 1 + src - first) * C + c];
        acc = fmaf(taps[(size_t)c * K + j], x, acc);
    }
    y[(size_t)n * C + c] = gd_silu(acc);
}

// The tails after the step: the last K - 1 of (old tail, the step's inputs).  One thread per
// (sequence, channel) reads its old entries before it writes.
__global__ __launch_bounds__(256) void conv_tail_kernel(
        const float* __restrict__ proj, int row_width, int K, int C, float* __restrict__ state,
        size_t slot_stride, size_t tail_off, const int* __restrict__ q_start,
        const int* __restrict__ slots, int n_seqs) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)n_seqs * C) return;
    const int b = (int)(idx / C), c = (int)(idx - (long long)b * C);
    const int first = q_start[b], L = q_start[b + 1] - first;
    float* tail = state + (size_t)slots[b] * slot_stride + tail_off;
    float old[GD_MAX_TAPS];
    for (int i = 0; i < K - 1; ++i) old[i] = tail[(size_t)i * C + c];
    for (int i = 0; i < K - 1; ++i) {
        const int at = L + i;                           // in (old tail, inputs of the step)
        tail[(size_t)i * C + c] = at < K - 1 ? old[at]
                                             : proj[(size_t)(first + at - (K - 1)) * row_width + c];
    }
}

extern "C" int gfa_short_conv(const float* proj, int row_width, const float* taps, int K, int C,
                              float* state, size_t slot_stride, size_t tail_off, const int* tok_seq,
                              const int* q_start, const int* slots, float* y, int n_tokens, int n_seqs,
                              hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (K < 1 || K > GD_MAX_TAPS || C < 1 || C > row_width) return (int)hipErrorInvalidValue;
    const long long units = (long long)n_tokens * C;
    short_conv_kernel<<<(unsigned)((units + 255) / 256), 256, 0, stream>>>(
        proj, row_width, taps, K, C, state, slot_stride, tail_off, tok_seq, q_start, slots, y, n_tokens);
    if (K > 1) {
        const long long tails = (long long)n_seqs * C;
        conv_tail_kernel<<<(unsigned)((tails + 255) / 256), 256, 0, stream>>>(
            proj, row_width, K, C, state, slot_stride, tail_off, q_start, slots, n_seqs);
    }
    return GFA_LAUNCH_RESULT();
}

struct GDShape {
    int H, G, dk, dv;
    int conv_width;                     // floats per row of the convolved q, k, v
    int row_width;                      // floats per row of proj
    int b_off, a_off;                   // columns of beta's and the decay's pre-activations in proj
    float q_scale, unit_eps;
};

// Token by token.  grid (dv / GD_COLS, H, sequences).  Thread (c, g) = (tid % 32, tid / 32)
// holds rows g, g + 8, ... of column c of S in registers.  With Sg = g S (the decayed state),
// a = Sg^T k', b = Sg^T q' and the three dot products k'.k', q'.q', k'.q' come from ONE pass
// over the thread's rows and one exchange through shared memory; with rk, rq the unit norms'
// factors:  u = beta (v - rk a),  S = Sg + rk k' u^T,  o = rq (b + rk (k'.q') u),
// which is S^T q after the write.  q', k' and the exchange buffer alternate between two
// copies, so a token costs two barriers; the next token's values are fetched meanwhile.
template <int RPT>
__global__ __launch_bounds__(GD_THREADS) void gated_delta_scan_kernel(
        const float* __restrict__ conv, const float* __restrict__ proj,
        const float* __restrict__ A_log, const float* __restrict__ dt_bias,
        float* __restrict__ state, size_t slot_stride, const int* __restrict__ q_start,
        const int* __restrict__ slots, float* __restrict__ out, GDShape s) {
    __shared__ float qs[2][RPT * GD_GROUPS], ks[2][RPT * GD_GROUPS];
    __shared__ float red[2][5][GD_GROUPS][GD_COLS];
    const int tid = threadIdx.x, c = tid % GD_COLS, g = tid / GD_COLS;
    const int col = blockIdx.x * GD_COLS + c;
    const int h = blockIdx.y, b = blockIdx.z;
    const int kvh = h / (s.H / s.G);
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const S = state + (size_t)slots[b] * slot_stride + (size_t)h * s.dk * s.dv;
    const bool col_ok = col < s.dv;
    const float rate = expf(A_log[h]), bias = dt_bias[h];
    const int q_col = kvh * s.dk, k_col = s.G * s.dk + kvh * s.dk, v_col = 2 * s.G * s.dk + h * s.dv;
    constexpr int EPT = (RPT * GD_GROUPS + GD_THREADS - 1) / GD_THREADS;   // elements of q a thread fetches

    float Sreg[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * GD_GROUPS;
        Sreg[r] = (col_ok && row < s.dk) ? S[(size_t)row * s.dv + col] : 0.f;
    }
    float nq[EPT], nk[EPT], nv = 0.f, nb = 0.f, na = 0.f;
    auto fetch = [&](int t) {
        const float* cr = conv + (size_t)t * s.conv_width;
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int e = tid + i * GD_THREADS;
            nq[i] = e < s.dk ? cr[q_col + e] : 0.f;
            nk[i] = e < s.dk ? cr[k_col + e] : 0.f;
        }
        nv = col_ok ? cr[v_col + col] : 0.f;
        const float* pr = proj + (size_t)t * s.row_width;
        nb = pr[s.b_off + h];
        na = pr[s.a_off + h];
    };
    if (t0 < t1) fetch(t0);
    for (int t = t0; t < t1; ++t) {
        const int p = (t - t0) & 1;
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int e = tid + i * GD_THREADS;
            if (e < RPT * GD_GROUPS) {
                qs[p][e] = nq[i];
                ks[p][e] = nk[i];
            }
        }
        const float v = nv;
        const float beta = 1.f / (1.f + expf(-nb));
        const float decay = expf(-rate * gd_softplus(na + bias));
        if (t + 1 < t1) fetch(t + 1);
        __syncthreads();
        float pa = 0.f, pb = 0.f, kk = 0.f, qq = 0.f, kq = 0.f;
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            const int e = g + r * GD_GROUPS;
            const float ke = ks[p][e], qe = qs[p][e];
            Sreg[r] *= decay;
            pa = fmaf(Sreg[r], ke, pa);
            pb = fmaf(Sreg[r], qe, pb);
            kk = fmaf(ke, ke, kk);
            qq = fmaf(qe, qe, qq);
            kq = fmaf(ke, qe, kq);
        }
        red[p][0][g][c] = pa;
        red[p][1][g][c] = pb;
        red[p][2][g][c] = kk;
        red[p][3][g][c] = qq;
        red[p][4][g][c] = kq;
        __syncthreads();
        float a = 0.f, bsum = 0.f;
        kk = qq = kq = 0.f;
#pragma unroll
        for (int r = 0; r < GD_GROUPS; ++r) {
            a += red[p][0][r][c];
            bsum += red[p][1][r][c];
            kk += red[p][2][r][c];
            qq += red[p][3][r][c];
            kq += red[p][4][r][c];
        }
        const float rk = rsqrtf(kk + s.unit_eps);
        const float rq = rsqrtf(qq + s.unit_eps) * s.q_scale;
        const float u = beta * (v - rk * a);
        const float ku = rk * u;
#pragma unroll
        for (int r = 0; r < RPT; ++r) Sreg[r] = fmaf(ks[p][g + r * GD_GROUPS], ku, Sreg[r]);
        if (g == 0 && col_ok)
            out[(size_t)t * s.H * s.dv + (size_t)h * s.dv + col] = rq * fmaf(rk * kq, u, bsum);
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * GD_GROUPS;
        if (col_ok && row < s.dk) S[(size_t)row * s.dv + col] = Sreg[r];
    }
}

extern "C" int gfa_gated_delta_scan(const float* conv, int conv_width, const float* proj, int row_width,
                                    int b_off, int a_off, const float* A_log, const float* dt_bias,
                                    float* state, size_t slot_stride, const int* q_start,
                                    const int* slots, float* out, int n_seqs, int H, int G, int dk,
                                    int dv, float q_scale, float unit_eps, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (dk < 1 || dk > 64 * GD_GROUPS || H < 1 || H > 65535 || G < 1 || H % G || n_seqs > 65535 ||
            conv_width < 2 * G * dk + H * dv || b_off + H > row_width || a_off + H > row_width)
        return (int)hipErrorInvalidValue;
    GDShape s{H, G, dk, dv, conv_width, row_width, b_off, a_off, q_scale, unit_eps};
    dim3 grid((dv + GD_COLS - 1) / GD_COLS, H, n_seqs);
    const int rpt = (dk + GD_GROUPS - 1) / GD_GROUPS;
#define GD_LAUNCH(R) gated_delta_scan_kernel<R><<<grid, GD_THREADS, 0, stream>>>( \
        conv, proj, A_log, dt_bias, state, slot_stride, q_start, slots, out, s)
    if (rpt <= 4) GD_LAUNCH(4);
    else if (rpt <= 8) GD_LAUNCH(8);
    else if (rpt <= 16) GD_LAUNCH(16);
    else if (rpt <= 32) GD_LAUNCH(32);
    else GD_LAUNCH(64);
#undef GD_LAUNCH
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The same cell for runs of many tokens, a chunk of 32 or 64 tokens at a time.  With S0 the state
// at the chunk's start, t, s = 0, 1, ... the chunk's tokens, G_t = sum_{r<=t} ln g_r and
// e(t, s) = exp(G_t - G_s) <= 1 for s <= t, the recurrence written out is
//     S_t = exp(G_t) S0 + sum_{s<=t} e(t, s) k_s u_s^T
//     u_t = beta_t (v_t - exp(G_t) S0^T k_t - sum_{s<t} e(t, s) (k_s . k_t) u_s)
// so the chunk's u solve (I + A) U = B with the strictly lower triangular
// A[t][s] = beta_t e(t, s) (k_t . k_s) and B_t = beta_t (v_t - exp(G_t) S0^T k_t): a forward
// substitution, row by row, eight threads to a column of the values.  Then
//     o_t = exp(G_t) S0^T q_t + sum_{s<=t} e(t, s) (k_s . q_t) u_s
//     S_L = exp(G_L) S0 + sum_s e(L, s) k_s u_s^T
// The products (K K^T, Q K^T, K S0, Q S0, P U, the state's update) run on the matrix cores in
// float (v_mfma_f32_16x16x4_f32: lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16] and
// holds C[4 (l / 16) .. +3][l % 16]).  grid (dv / GC_COLS, H, sequences), eight threads per token
// of a chunk; the chunk's unit q and k, v, A, the weighted scores P, U and the workgroup's
// columns of S are in shared memory.
#define GC_COLS 32
#define GC_BLOCK 32                     // rows of the substitution that eight threads a column take at once

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float gc_floatx4_t;

__host__ __device__ inline int gc_padded(int dk) { return (dk + 15) / 16 * 16; }
__host__ __device__ inline int gc_row_stride(int dk) { return gc_padded(dk) + 4; }

// GC_L: tokens per chunk (32 or 64), eight threads per token; NV: 16-byte loads of q and of k
// per thread (0: plain loads).  A chunk of 64 solves (I + A) U = B in two blocks of 32 rows:
// the first by substitution, then B_2 - A_21 U_1 on the matrix cores, then the second.
template <int GC_L, int NV>
__global__ __launch_bounds__(GC_L * 8) void gated_delta_chunk_kernel(
        const float* __restrict__ conv, const float* __restrict__ proj,
        const float* __restrict__ A_log, const float* __restrict__ dt_bias,
        float* __restrict__ state, size_t slot_stride, const int* __restrict__ q_start,
        const int* __restrict__ slots, float* __restrict__ out, GDShape s) {
    extern __shared__ __attribute__((aligned(16))) float gc_lds[];
    constexpr int NT = GC_L * 8, NW = NT / 64, GC_PS = GC_L + 1;
    const int KS = gc_row_stride(s.dk), dkp = gc_padded(s.dk);
    float* Qs = gc_lds;                          // [GC_L][KS]  unit q times q_scale
    float* Ks = Qs + GC_L * KS;                  // [GC_L][KS]  unit k
    float* Vs = Ks + GC_L * KS;                  // [GC_L][GC_COLS]
    float* Us = Vs + GC_L * GC_COLS;             // [GC_L][GC_COLS]  B, then U
    float* As = Us + GC_L * GC_COLS;             // [GC_L][GC_PS]
    float* Ps = As + GC_L * GC_PS;               // [GC_L][GC_PS]
    float* Ss = Ps + GC_L * GC_PS;               // [dkp][GC_COLS]
    float* gam = Ss + dkp * GC_COLS;             // [GC_L]  G_t
    float* bet = gam + GC_L;                     // [GC_L]
    float* wl = bet + GC_L;                      // [GC_L]  e(L, s), 0 beyond the chunk's end
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col0 = blockIdx.x * GC_COLS;
    const int h = blockIdx.y, b = blockIdx.z;
    const int kvh = h / (s.H / s.G);
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const S = state + (size_t)slots[b] * slot_stride + (size_t)h * s.dk * s.dv;
    const float rate = expf(A_log[h]), bias = dt_bias[h];
    const int q_col = kvh * s.dk, k_col = s.G * s.dk + kvh * s.dk, v_col = 2 * s.G * s.dk + h * s.dv;

    for (int e = tid; e < dkp * GC_COLS; e += NT) {
        const int d = e / GC_COLS, c = e % GC_COLS;
        Ss[e] = (d < s.dk && col0 + c < s.dv) ? S[(size_t)d * s.dv + col0 + c] : 0.f;
    }
    for (int e = tid; e < 2 * GC_L * KS; e += NT) Qs[e] = 0.f;       // q and k: the filling stays zero
    for (int e = tid; e < GC_L * GC_PS; e += NT) As[e] = 0.f;        // the tiles above the diagonal stay zero

    const int li = lane & 15, lg = lane >> 4;
    // eight threads per token fetch its q and k (16 bytes at a time where NV > 0: the rows'
    // sizes and offsets are then multiples of four) and its values a chunk ahead, into registers
    const int ft = tid >> 3, sub = tid & 7;
    const int n4 = s.dk >> 2;
    float4 rq[NV > 0 ? NV : 1], rk[NV > 0 ? NV : 1];
    float rv[4], rb = 0.f, ra = 0.f;
    auto fetch = [&](int c0) {
        const int Lc = t1 - c0 < GC_L ? t1 - c0 : GC_L;
        const bool live = ft < Lc;
        const float* cr = conv + (size_t)(c0 + (live ? ft : 0)) * s.conv_width;
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int j = sub + 8 * i;
            const bool in = live && j < n4;
            rq[i] = in ? *(const float4*)(cr + q_col + 4 * j) : zero;
            rk[i] = in ? *(const float4*)(cr + k_col + 4 * j) : zero;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = sub * 4 + i;
            rv[i] = (live && col0 + c < s.dv) ? cr[v_col + col0 + c] : 0.f;
        }
        if (tid < GC_L) {
            const bool mine = tid < Lc;
            const float* pr = proj + (size_t)(c0 + (mine ? tid : 0)) * s.row_width;
            rb = mine ? pr[s.b_off + h] : 0.f;
            ra = mine ? pr[s.a_off + h] : 0.f;
        }
    };
    if (t0 < t1) fetch(t0);
    for (int c0 = t0; c0 < t1; c0 += GC_L) {
        const int Lc = t1 - c0 < GC_L ? t1 - c0 : GC_L;
        __syncthreads();                         // the chunk before is done with everything
        {
            // the token's q and k as unit vectors, its values
            const bool live = ft < Lc;
            float sq = 0.f, sk = 0.f;
            if (NV > 0) {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    sq += rq[i].x * rq[i].x + rq[i].y * rq[i].y + rq[i].z * rq[i].z + rq[i].w * rq[i].w;
                    sk += rk[i].x * rk[i].x + rk[i].y * rk[i].y + rk[i].z * rk[i].z + rk[i].w * rk[i].w;
                }
            } else if (live) {
                const float* cr = conv + (size_t)(c0 + ft) * s.conv_width;
                for (int e = sub; e < s.dk; e += 8) {
                    const float qv = cr[q_col + e], kv = cr[k_col + e];
                    sq = fmaf(qv, qv, sq);
                    sk = fmaf(kv, kv, sk);
                }
            }
#pragma unroll
            for (int o = 1; o < 8; o <<= 1) {
                sq += __shfl_xor(sq, o, 64);
                sk += __shfl_xor(sk, o, 64);
            }
            const float fq = rsqrtf(sq + s.unit_eps) * s.q_scale, fk = rsqrtf(sk + s.unit_eps);
            if (NV > 0) {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int j = sub + 8 * i;
                    if (j < n4) {
                        *(float4*)(Qs + ft * KS + 4 * j) =
                            make_float4(rq[i].x * fq, rq[i].y * fq, rq[i].z * fq, rq[i].w * fq);
                        *(float4*)(Ks + ft * KS + 4 * j) =
                            make_float4(rk[i].x * fk, rk[i].y * fk, rk[i].z * fk, rk[i].w * fk);
                    }
                }
            } else {
                const float* cr = conv + (size_t)(c0 + (live ? ft : 0)) * s.conv_width;
                for (int e = sub; e < s.dk; e += 8) {
                    Qs[ft * KS + e] = live ? cr[q_col + e] * fq : 0.f;
                    Ks[ft * KS + e] = live ? cr[k_col + e] * fk : 0.f;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) Vs[ft * GC_COLS + sub * 4 + i] = rv[i];
        }
        if (tid < 64) {
            // the first wave: beta, and the running sum of the log decays over its lanes
            const bool mine = tid < Lc;
            float run = mine ? -rate * gd_softplus(ra + bias) : 0.f;
#pragma unroll
            for (int o = 1; o < GC_L; o <<= 1) {
                const float up = __shfl_up(run, o, 64);
                if (tid >= o) run += up;
            }
            const float last = __shfl(run, GC_L - 1, 64);
            if (tid < GC_L) {
                bet[tid] = mine ? 1.f / (1.f + expf(-rb)) : 0.f;
                gam[tid] = run;
                wl[tid] = mine ? expf(last - run) : 0.f;
            }
        }
        if (c0 + GC_L < t1) fetch(c0 + GC_L);
        __syncthreads();
        // k.k and q.k of the chunk, decayed: the 16 x 16 tiles on and below the diagonal, first
        // those of A, then those of P, handed out over the waves
        constexpr int LOWER = (GC_L / 16) * (GC_L / 16 + 1) / 2;
        for (int idx = wave; idx < 2 * LOWER; idx += NW) {
            const bool is_p = idx >= LOWER;
            const int tile = is_p ? idx - LOWER : idx;
            int ti = 0;
            while ((ti + 1) * (ti + 2) / 2 <= tile) ++ti;
            const int si = tile - ti * (ti + 1) / 2;
            gc_floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
            const float* ra_ = (is_p ? Qs : Ks) + (ti * 16 + li) * KS + lg;
            const float* kb = Ks + (si * 16 + li) * KS + lg;
#pragma unroll 4
            for (int d0 = 0; d0 < dkp; d0 += 4)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ra_[d0], kb[d0], acc, 0, 0, 0);
            const int ss = si * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = ti * 16 + lg * 4 + r;
                const float e = ss <= t ? expf(gam[t] - gam[ss]) : 0.f;
                if (is_p) Ps[t * GC_PS + ss] = acc[r] * e;
                else As[t * GC_PS + ss] = ss < t ? bet[t] * acc[r] * e : 0.f;
            }
        }
        // the state's share: B = beta (V - exp(G) K S0) into Us, and exp(G) Q S0 kept for o
        gc_floatx4_t num = {0.f, 0.f, 0.f, 0.f};
        const int oti = wave >> 1, oci = wave & 1;
        {
            gc_floatx4_t ks0 = {0.f, 0.f, 0.f, 0.f};
            const float* qa = Qs + (oti * 16 + li) * KS + lg;
            const float* ka = Ks + (oti * 16 + li) * KS + lg;
            const float* sb = Ss + lg * GC_COLS + oci * 16 + li;
#pragma unroll 4
            for (int d0 = 0; d0 < dkp; d0 += 4) {
                num = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[d0], sb[d0 * GC_COLS], num, 0, 0, 0);
                ks0 = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[d0], sb[d0 * GC_COLS], ks0, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = oti * 16 + lg * 4 + r, c = oci * 16 + li;
                const float eg = expf(gam[t]);
                num[r] *= eg;
                Us[t * GC_COLS + c] = bet[t] * (Vs[t * GC_COLS + c] - eg * ks0[r]);
            }
        }
        __syncthreads();                         // As, Ps and B are whole
#pragma unroll
        for (int blk = 0; blk < GC_L / GC_BLOCK; ++blk) {
            const int r0 = blk * GC_BLOCK;
            if (blk > 0) {
                // the rows of this block take off what the rows before them add: B - A U on the
                // matrix cores, a 16 x 16 tile per wave of the first four
                if (wave < 4) {
                    const int bi = wave >> 1, bc = wave & 1;
                    gc_floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
                    const float* aa = As + (r0 + bi * 16 + li) * GC_PS + lg;
                    const float* ub = Us + lg * GC_COLS + bc * 16 + li;
                    for (int s0 = 0; s0 < r0; s0 += 4)
                        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aa[s0], ub[s0 * GC_COLS], acc, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        Us[(r0 + bi * 16 + lg * 4 + r) * GC_COLS + bc * 16 + li] -= acc[r];
                }
                __syncthreads();
            }
            if (tid < 8 * GC_COLS) {
                // (I + A) U = B row by row within the block: eight threads per column of the
                // values, thread g of them keeps u_s for s = g, g + 8, ... and adds its share of
                // sum_s A[t][s] u_s; entries of A on and above the diagonal are zero, and so are
                // the u not yet known
                const int c = tid >> 3, g = tid & 7;
                float ureg[GC_BLOCK / 8];
#pragma unroll
                for (int i = 0; i < GC_BLOCK / 8; ++i) ureg[i] = 0.f;
#pragma unroll
                for (int t = 0; t < GC_BLOCK; ++t) {
                    float part = 0.f;
#pragma unroll
                    for (int i = 0; i < GC_BLOCK / 8; ++i)
                        part = fmaf(As[(r0 + t) * GC_PS + r0 + g + 8 * i], ureg[i], part);
                    part += __shfl_xor(part, 1, 64);
                    part += __shfl_xor(part, 2, 64);
                    part += __shfl_xor(part, 4, 64);
                    const float ut = Us[(r0 + t) * GC_COLS + c] - part;
                    if (g == (t & 7)) ureg[t >> 3] = ut;
                    if (g == 0) Us[(r0 + t) * GC_COLS + c] = ut;
                }
            }
            __syncthreads();                     // the block's U is whole
        }
        {
            const float* pa = Ps + (oti * 16 + li) * GC_PS + lg;
            const float* ub = Us + lg * GC_COLS + oci * 16 + li;
#pragma unroll 4
            for (int s0 = 0; s0 < (oti + 1) * 16; s0 += 4)
                num = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[s0], ub[s0 * GC_COLS], num, 0, 0, 0);
            const int c = col0 + oci * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = oti * 16 + lg * 4 + r;
                if (t < Lc && c < s.dv)
                    out[(size_t)(c0 + t) * s.H * s.dv + (size_t)h * s.dv + c] = num[r];
            }
        }
        // the state after the chunk's last token: S = exp(G_L) S + (w K)^T U, a wave's tiles of
        // 16 rows of S by 16 columns in turn (every wave has read S0 before the barriers above)
        {
            const float aL = expf(gam[GC_L - 1]);
            for (int tile = wave; tile < (dkp / 16) * 2; tile += NW) {
                const int di = tile >> 1, ci = tile & 1;
                float* sc = Ss + (di * 16 + lg * 4) * GC_COLS + ci * 16 + li;
                gc_floatx4_t acc;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = aL * sc[r * GC_COLS];
                const float* ka = Ks + lg * KS + di * 16 + li;
                const float* ub = Us + lg * GC_COLS + ci * 16 + li;
#pragma unroll
                for (int s0 = 0; s0 < GC_L; s0 += 4)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wl[s0 + lg] * ka[s0 * KS], ub[s0 * GC_COLS],
                                                              acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) sc[r * GC_COLS] = acc[r];
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < s.dk * GC_COLS; e += NT) {
        const int d = e / GC_COLS, c = e % GC_COLS;
        if (col0 + c < s.dv) S[(size_t)d * s.dv + col0 + c] = Ss[e];
    }
}

static int gc_lds_bytes(int dk, int L) {
    return (int)sizeof(float) * (2 * L * gc_row_stride(dk) + 2 * L * GC_COLS + 2 * L * (L + 1)
                                 + gc_padded(dk) * GC_COLS + 3 * L);
}

static int gc_lds_limit() {
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

static bool gc_fits(int dk, int L) {
    const int bytes = gc_lds_bytes(dk, L);
    return bytes <= gc_lds_limit() && bytes <= 160 * 1024;
}

// 1 if the chunked kernel takes these sizes on this device
extern "C" int gfa_gated_delta_chunks_take(int dk, int dv) {
    return dk >= 1 && dv >= 1 && gc_fits(dk, 32) ? 1 : 0;
}

template <int L, int NV>
static int gc_launch(const float* conv, const float* proj, const float* A_log, const float* dt_bias,
                     float* state, size_t slot_stride, const int* q_start, const int* slots, float* out,
                     const GDShape& s, dim3 grid, hipStream_t stream) {
    const int bytes = gc_lds_bytes(s.dk, L);
    if (bytes > 64 * 1024) {
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute((const void*)gated_delta_chunk_kernel<L, NV>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
    }
    gated_delta_chunk_kernel<L, NV><<<grid, L * 8, bytes, stream>>>(conv, proj, A_log, dt_bias, state,
                                                                    slot_stride, q_start, slots, out, s);
    return GFA_LAUNCH_RESULT();
}

// Chunks of 64 tokens (512 threads) where the device lets a workgroup have the shared memory for
// them and some sequence brings that many, else chunks of 32 (256 threads): a longer chunk
// spreads the chain of barriers and the state's products over twice the tokens.
extern "C" int gfa_gated_delta_chunks(const float* conv, int conv_width, const float* proj, int row_width,
                                      int b_off, int a_off, const float* A_log, const float* dt_bias,
                                      float* state, size_t slot_stride, const int* q_start,
                                      const int* slots, float* out, int n_seqs, int max_q_len, int H,
                                      int G, int dk, int dv, float q_scale, float unit_eps,
                                      hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (dk < 1 || H < 1 || H > 65535 || G < 1 || H % G || n_seqs > 65535 ||
            conv_width < 2 * G * dk + H * dv || b_off + H > row_width || a_off + H > row_width ||
            !gfa_gated_delta_chunks_take(dk, dv))
        return (int)hipErrorInvalidValue;
    GDShape s{H, G, dk, dv, conv_width, row_width, b_off, a_off, q_scale, unit_eps};
    dim3 grid((dv + GC_COLS - 1) / GC_COLS, H, n_seqs);
    // 16-byte loads of q and k where every row and head starts at a multiple of four floats
    const bool vec = dk % 4 == 0 && conv_width % 4 == 0 && (size_t)conv % 16 == 0 && dk <= 256;
    const bool big = max_q_len > 32 && gc_fits(dk, 64);
#define GC_GO(NV) return big ? gc_launch<64, NV>(conv, proj, A_log, dt_bias, state, slot_stride, q_start, \
                                                 slots, out, s, grid, stream) \
                             : gc_launch<32, NV>(conv, proj, A_log, dt_bias, state, slot_stride, q_start, \
                                                 slots, out, s, grid, stream)
    if (!vec) GC_GO(0);
    if (dk <= 64) GC_GO(2);
    if (dk <= 128) GC_GO(4);
    GC_GO(8);
#undef GC_GO
}
