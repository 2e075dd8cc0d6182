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
