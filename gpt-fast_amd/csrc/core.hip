// Plain kernels for every op of a decoder step.
//
// These are the reference kernels of the library: simple, one workgroup per row or per
// (token, head), all arithmetic in float.  The float32 engine runs on them alone; the
// bfloat16 engine uses them where no faster kernel exists, and the faster kernels are
// tested against them.  In each kernel the order of floating-point additions that
// produce one output element depends only on that element's own inputs (its row, its
// position), never on the number of rows or on the other sequences of the launch, so a
// float32 result is the same however the tokens were cut into steps or batched.
#include "common.h"

// --------------------------------------------------------------------------------------
// embedding gather: out[n, :] = float(table[tokens[n], :])          (model.py:140)
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ out, int dim) {
    const int n = blockIdx.x;
    const T* row = table + (size_t)tokens[n] * dim;
    float* o = out + (size_t)n * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] = load_as_float(row + d);
}

extern "C" int gfa_embed(const void* table, int table_bf16, const int* tokens, float* out,
                         int n_tokens, int dim, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (table_bf16)
        embed_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)table, tokens, out, dim);
    else
        embed_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, tokens, out, dim);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// RMS norm: out[i, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w[:],  r = rows ? rows[i] : i
// (model.py:236-241; statistics in float, one rounding at the store)
template <typename T>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               const int* __restrict__ rows, T* __restrict__ out, int dim,
                               float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    const float* xr = x + (size_t)r * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = xr[d];
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    T* o = out + (size_t)i * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) store_from_float(o + d, xr[d] * rs * w[d]);
}

// The same for rows of up to 1024 * VPT elements (a multiple of 4): the row is read once
// with 16-byte loads, kept in registers between the sum and the scaling.
template <typename T, int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_vec_kernel(
        const float* __restrict__ x, const float* __restrict__ w, const int* __restrict__ rows,
        T* __restrict__ out, int dim, float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    const float4* xr = (const float4*)(x + (size_t)r * dim);
    const float4* w4 = (const float4*)w;
    const int n4 = dim >> 2;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        v[j] = idx < n4 ? xr[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
        ss = fmaf(v[j].x, v[j].x, ss);
        ss = fmaf(v[j].y, v[j].y, ss);
        ss = fmaf(v[j].z, v[j].z, ss);
        ss = fmaf(v[j].w, v[j].w, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    T* o = out + (size_t)i * dim;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = w4[idx];
            store_from_float(o + 4 * idx + 0, v[j].x * rs * g.x);
            store_from_float(o + 4 * idx + 1, v[j].y * rs * g.y);
            store_from_float(o + 4 * idx + 2, v[j].z * rs * g.z);
            store_from_float(o + 4 * idx + 3, v[j].w * rs * g.w);
        }
    }
}

template <typename T>
static bool launch_rmsnorm_vec(const float* x, const float* w, const int* rows, T* out, int n_rows,
                               int dim, float eps, hipStream_t stream) {
    if (dim % 4 != 0 || dim > 8192) return false;
    // one float4 per thread where the row allows it: the kernel is a chain of latencies
    if (dim <= 1024) rmsnorm_vec_kernel<T, 1, 256><<<n_rows, 256, 0, stream>>>(x, w, rows, out, dim, eps);
    else if (dim <= 4096) rmsnorm_vec_kernel<T, 1, 1024><<<n_rows, 1024, 0, stream>>>(x, w, rows, out, dim, eps);
    else rmsnorm_vec_kernel<T, 2, 1024><<<n_rows, 1024, 0, stream>>>(x, w, rows, out, dim, eps);
    return true;
}

extern "C" int gfa_rmsnorm(const float* x, const float* w, const int* rows, void* out,
                           int out_bf16, int n_rows, int dim, float eps, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (out_bf16 ? launch_rmsnorm_vec<bf16_t>(x, w, rows, (bf16_t*)out, n_rows, dim, eps, stream)
                 : launch_rmsnorm_vec<float>(x, w, rows, (float*)out, n_rows, dim, eps, stream))
        return GFA_LAUNCH_RESULT();
    if (out_bf16)
        rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, w, rows, (bf16_t*)out, dim, eps);
    else
        rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>(x, w, rows, (float*)out, dim, eps);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The sum that completes a block and the norm that opens the next, one pass over each row:
// res[i, :] += float(y[i, :]);  out[i, :] = rmsnorm(res[i, :]) in bfloat16
// (model.py:162-163 followed by 236-241; the sum and the statistics in float)
__global__ void add_rmsnorm_kernel(float* __restrict__ res, const bf16_t* __restrict__ y,
                                   const float* __restrict__ w, bf16_t* __restrict__ out, int dim,
                                   float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    float* xr = res + (size_t)i * dim;
    const bf16_t* yr = y + (size_t)i * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        const float v = xr[d] + bf16_to_float(yr[d]);
        xr[d] = v;                                       // read back by this thread only
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    bf16_t* o = out + (size_t)i * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) store_from_float(o + d, xr[d] * rs * w[d]);
}

// rows of up to 1024 * VPT elements (a multiple of 4), kept in registers
template <int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_vec_kernel(
        float* __restrict__ res, const bf16_t* __restrict__ y, const float* __restrict__ w,
        bf16_t* __restrict__ out, int dim, float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    float4* xr = (float4*)(res + (size_t)i * dim);
    const uint2* yr = (const uint2*)(y + (size_t)i * dim);
    const float4* w4 = (const float4*)w;
    const int n4 = dim >> 2;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (idx < n4) {
            v[j] = xr[idx];
            const uint2 a = yr[idx];
            v[j].x += __uint_as_float(a.x << 16);
            v[j].y += __uint_as_float(a.x & 0xffff0000u);
            v[j].z += __uint_as_float(a.y << 16);
            v[j].w += __uint_as_float(a.y & 0xffff0000u);
            xr[idx] = v[j];
        }
        ss = fmaf(v[j].x, v[j].x, ss);
        ss = fmaf(v[j].y, v[j].y, ss);
        ss = fmaf(v[j].z, v[j].z, ss);
        ss = fmaf(v[j].w, v[j].w, ss);
    }
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)dim + eps);
    uint2* o = (uint2*)(out + (size_t)i * dim);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = w4[idx];
            bf16_t e[4];
            e[0] = float_to_bf16(v[j].x * rs * g.x);
            e[1] = float_to_bf16(v[j].y * rs * g.y);
            e[2] = float_to_bf16(v[j].z * rs * g.z);
            e[3] = float_to_bf16(v[j].w * rs * g.w);
            o[idx] = make_uint2((unsigned)e[0] | ((unsigned)e[1] << 16),
                                (unsigned)e[2] | ((unsigned)e[3] << 16));
        }
    }
}

extern "C" int gfa_add_rmsnorm(float* res, const void* y, const float* w, void* out, int n_rows,
                               int dim, float eps, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    const bf16_t* yp = (const bf16_t*)y;
    bf16_t* op = (bf16_t*)out;
    const bool vec = dim % 4 == 0 && dim <= 8192 && (uintptr_t)res % 16 == 0 &&
                     (uintptr_t)y % 8 == 0 && (uintptr_t)out % 8 == 0 && (uintptr_t)w % 16 == 0;
    if (!vec) add_rmsnorm_kernel<<<n_rows, 256, 0, stream>>>(res, yp, w, op, dim, eps);
    else if (dim <= 1024) add_rmsnorm_vec_kernel<1, 256><<<n_rows, 256, 0, stream>>>(res, yp, w, op, dim, eps);
    else if (dim <= 4096) add_rmsnorm_vec_kernel<1, 1024><<<n_rows, 1024, 0, stream>>>(res, yp, w, op, dim, eps);
    else add_rmsnorm_vec_kernel<2, 1024><<<n_rows, 1024, 0, stream>>>(res, yp, w, op, dim, eps);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// float32 matrix product: out[m, n] (+)= sum_k a[m, k] * w[n, k]
// 64x64 tile per workgroup of 256 threads, 4x4 outputs per thread, k in steps of 16 through
// shared memory.  Each output is one fused-multiply-add chain over k = 0..K-1 in order.
#define GF_BM 64
#define GF_BN 64
#define GF_BK 16
__global__ __launch_bounds__(256) void gemm_f32_kernel(
        const float* __restrict__ a, const float* __restrict__ w, float* __restrict__ out,
        int M, int N, int K, int lda, int ldo, int accumulate) {
    __shared__ float As[GF_BK][GF_BM + 4];
    __shared__ float Ws[GF_BK][GF_BN + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GF_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = threadIdx.x + i * 256;
            const int r = e >> 4, c = e & 15;
            const int k = k0 + c;
            const int m = m0 + r, n = n0 + r;
            As[c][r] = (m < M && k < K) ? a[(size_t)m * lda + k] : 0.f;
            Ws[c][r] = (n < N && k < K) ? w[(size_t)n * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GF_BK; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float* o = out + (size_t)m * ldo + n;
            *o = accumulate ? (*o + acc[i][j]) : acc[i][j];
        }
    }
}

extern "C" int gfa_gemm_f32(const float* a, const float* w, float* out, int M, int N, int K,
                            int lda, int ldo, int accumulate, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM);
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, w, out, M, N, K, lda, ldo, accumulate);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Rotary position encoding of q and k, and the write of k and v into the paged cache.
// qkv: [N, (H + 2*Hkv) * hd] rows of q heads, k heads, v heads (model.py:195-199).
// Pair i of a head is (2i, 2i+1) if layout == 0 (model.py:281-293) or (i, i + rot/2) if
// layout == 1; it is rotated by angle = float(position) * freqs[i], cos and sin in float.
// Elements beyond `rot` pass through.  q goes to q_out [N, H, hd]; k and v of token n go
// to page table[seq(n)][pos / PAGE], offset pos % PAGE (model.py:91-100, 206-207); keys as
// rows [offset, hd], values transposed [hd, offset] (see common.h).
template <typename T>
__global__ __launch_bounds__(256) void rope_cache_kernel(
        const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_pages,
        T* __restrict__ v_pages, const float* __restrict__ freqs, const int* __restrict__ tok_seq,
        const int* __restrict__ tok_pos, const int* __restrict__ table, int table_stride, int H,
        int Hkv, int hd, int rot, int layout) {
    // one thread per pair of elements: q and k heads first (rotated or passed through), then
    // the pairs of v; blockIdx.y walks the token's pairs in groups of 256
    const int n = blockIdx.x;
    const int half = hd / 2;
    const int rot_pairs = rot / 2;
    const int qk_slots = (H + Hkv) * half, v_slots = Hkv * half;
    const int pos = tok_pos[n];
    // cos and sin of this token's angles, once per workgroup
    extern __shared__ float cs[];                          // [rot_pairs][2]
    if (blockIdx.y * 256 < qk_slots) {
        for (int i = threadIdx.x; i < rot_pairs; i += 256)
            sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
        __syncthreads();
    }
    const int e = blockIdx.y * 256 + threadIdx.x;
    if (e >= qk_slots + v_slots) return;
    const T* row = qkv + (size_t)n * (H + 2 * Hkv) * hd;
    int page = 0;
    if (k_pages) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    if (e < qk_slots) {
        const int head = e / half, i = e - head * half;
        const T* src = row + (size_t)head * hd;
        if (head >= H && !k_pages) return;
        // where element d of this head goes: a row of q_out, or the key's place in its page
        T* const dst = head < H ? q_out + ((size_t)n * H + head) * hd
                                : k_pages + cache_region(page, head - H, Hkv, hd);
        auto place = [&](int d) { return head < H ? d : key_offset(off, d, hd); };
        if (i < rot_pairs) {
            const int ia = layout == 0 ? 2 * i : i;
            const int ib = layout == 0 ? 2 * i + 1 : i + rot_pairs;
            const float a = load_as_float(src + ia), b = load_as_float(src + ib);
            const float c = cs[2 * i], s = cs[2 * i + 1];
            store_from_float(dst + place(ia), a * c - b * s);
            store_from_float(dst + place(ib), b * c + a * s);
        } else {
            const int d0 = rot + 2 * (i - rot_pairs);      // elements rot .. hd-1 are copied
            dst[place(d0)] = src[d0];
            dst[place(d0 + 1)] = src[d0 + 1];
        }
    } else if (v_pages) {
        const int ev = e - qk_slots;
        const int g = ev / half, d = 2 * (ev - g * half);
        const T* vsrc = row + (size_t)(H + Hkv + g) * hd + d;
        v_pages[value_elem(page, g, d, off, Hkv, hd)] = vsrc[0];
        v_pages[value_elem(page, g, d + 1, off, Hkv, hd)] = vsrc[1];
    }
}

// The same for bfloat16 with interleaved pairs, eight elements (four pairs) per thread:
// 16-byte loads and stores for q and k.  Needs hd and rot to be multiples of 8.
__global__ __launch_bounds__(256) void rope_cache_bf16x8_kernel(
        const bf16_t* __restrict__ qkv, bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_pages,
        bf16_t* __restrict__ v_pages, const float* __restrict__ freqs,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, int H, int Hkv, int hd, int rot) {
    const int n = blockIdx.x;
    const int per_head = hd / 8;
    const int qk_chunks = (H + Hkv) * per_head, v_chunks = Hkv * per_head;
    const int pos = tok_pos[n];
    extern __shared__ float cs[];                          // [rot / 2][2]
    if (blockIdx.y * 256 < qk_chunks) {
        for (int i = threadIdx.x; i < rot / 2; i += 256)
            sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
        __syncthreads();
    }
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= qk_chunks + v_chunks) return;
    const int head = c / per_head, d0 = (c - head * per_head) * 8;
    union { uint4 u; bf16_t e[8]; } in, out;
    in.u = *(const uint4*)(qkv + ((size_t)n * (H + 2 * Hkv) + head) * hd + d0);
    int page = 0;
    if (k_pages && head >= H) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    if (head < H + Hkv) {
        if (d0 < rot) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float a = bf16_to_float(in.e[2 * p]), b = bf16_to_float(in.e[2 * p + 1]);
                const float c_ = cs[d0 + 2 * p], s_ = cs[d0 + 2 * p + 1];
                out.e[2 * p] = float_to_bf16(a * c_ - b * s_);
                out.e[2 * p + 1] = float_to_bf16(b * c_ + a * s_);
            }
        } else {
            out.u = in.u;
        }
        if (head < H) {
            *(uint4*)(q_out + ((size_t)n * H + head) * hd + d0) = out.u;
        } else if (k_pages) {
            *(uint4*)(k_pages + key_elem(page, head - H, off, d0, Hkv, hd)) = out.u;   // one chunk of 8 dims
        }
    } else if (v_pages) {
        const int g = head - H - Hkv;
#pragma unroll
        for (int j = 0; j < 8; ++j) v_pages[value_elem(page, g, d0 + j, off, Hkv, hd)] = in.e[j];
    }
}

// The same with the rows given as float partial sums of a sliced product, part [S, N, width]:
// the slices are added in order (the sum a kernel of its own would form), rotated and stored,
// so that the product's second kernel is this one.  The rotation then works on the float sums
// instead of their bfloat16 rounding.
__global__ __launch_bounds__(256) void rope_cache_sliced_bf16x8_kernel(
        const float* __restrict__ part, int S, size_t slice, bf16_t* __restrict__ q_out,
        bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const float* __restrict__ freqs,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, int H, int Hkv, int hd, int rot) {
    const int n = blockIdx.x;
    const int per_head = hd / 8;
    const int qk_chunks = (H + Hkv) * per_head, v_chunks = Hkv * per_head;
    const int pos = tok_pos[n];
    extern __shared__ float cs[];                          // [rot / 2][2]
    if (blockIdx.y * 256 < qk_chunks) {
        for (int i = threadIdx.x; i < rot / 2; i += 256)
            sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
        __syncthreads();
    }
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= qk_chunks + v_chunks) return;
    const int head = c / per_head, d0 = (c - head * per_head) * 8;
    const float* src = part + ((size_t)n * (H + 2 * Hkv) + head) * hd + d0;
    float v[8];
    {
        const float4 a = *(const float4*)src, b = *(const float4*)(src + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    for (int s = 1; s < S; ++s) {
        const float4 a = *(const float4*)(src + s * slice), b = *(const float4*)(src + s * slice + 4);
        v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
    }
    int page = 0;
    if (k_pages && head >= H) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    union { uint4 u; bf16_t e[8]; } out;
    if (head < H + Hkv) {
        if (d0 < rot) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float a = v[2 * p], b = v[2 * p + 1];
                const float c_ = cs[d0 + 2 * p], s_ = cs[d0 + 2 * p + 1];
                out.e[2 * p] = float_to_bf16(a * c_ - b * s_);
                out.e[2 * p + 1] = float_to_bf16(b * c_ + a * s_);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) out.e[j] = float_to_bf16(v[j]);
        }
        if (head < H) {
            *(uint4*)(q_out + ((size_t)n * H + head) * hd + d0) = out.u;
        } else if (k_pages) {
            *(uint4*)(k_pages + key_elem(page, head - H, off, d0, Hkv, hd)) = out.u;
        }
    } else if (v_pages) {
        const int g = head - H - Hkv;
#pragma unroll
        for (int j = 0; j < 8; ++j) v_pages[value_elem(page, g, d0 + j, off, Hkv, hd)] = float_to_bf16(v[j]);
    }
}

// part [S, n_tokens, (H + 2 Hkv) * hd] float; interleaved pairs, hd and rot multiples of 8.
extern "C" int gfa_rope_cache_write_sliced(const float* part, int S, void* q_out, void* k_pages,
                                           void* v_pages, const float* freqs, const int* tok_seq,
                                           const int* tok_pos, const int* table, int table_stride,
                                           int n_tokens, int H, int Hkv, int hd, int rot,
                                           hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (S <= 0 || hd % 8 != 0 || rot % 8 != 0 || rot > hd || (rot > 0 && !freqs))
        return (int)hipErrorInvalidValue;
    const dim3 grid(n_tokens, ((H + 2 * Hkv) * (hd / 8) + 255) / 256);
    const size_t slice = (size_t)n_tokens * (H + 2 * Hkv) * hd;
    rope_cache_sliced_bf16x8_kernel<<<grid, 256, (size_t)(rot > 0 ? rot : 2) * sizeof(float), stream>>>(
        part, S, slice, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, freqs, tok_seq, tok_pos,
        table, table_stride, H, Hkv, hd, rot);
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_rope_cache_write(const void* qkv, void* q_out, void* k_pages, void* v_pages,
                                    const float* freqs, const int* tok_seq, const int* tok_pos,
                                    const int* table, int table_stride, int n_tokens, int H,
                                    int Hkv, int hd, int rot, int layout, int is_bf16,
                                    hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (is_bf16 && layout == 0 && hd % 8 == 0 && rot % 8 == 0) {
        const dim3 grid8(n_tokens, ((H + 2 * Hkv) * (hd / 8) + 255) / 256);
        rope_cache_bf16x8_kernel<<<grid8, 256, (size_t)(rot > 0 ? rot : 2) * sizeof(float), stream>>>(
            (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, freqs, tok_seq,
            tok_pos, table, table_stride, H, Hkv, hd, rot);
        return GFA_LAUNCH_RESULT();
    }
    const dim3 grid(n_tokens, ((H + 2 * Hkv) * (hd / 2) + 255) / 256);
    if (is_bf16)
        rope_cache_kernel<bf16_t><<<grid, 256, (size_t)rot * sizeof(float), stream>>>(
            (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, freqs,
            tok_seq, tok_pos, table, table_stride, H, Hkv, hd, rot, layout);
    else
        rope_cache_kernel<float><<<grid, 256, (size_t)rot * sizeof(float), stream>>>(
            (const float*)qkv, (float*)q_out, (float*)k_pages, (float*)v_pages, freqs, tok_seq,
            tok_pos, table, table_stride, H, Hkv, hd, rot, layout);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Attention of each new token over its sequence's cache (model.py:209-211 with the mask of
// model.py:134,138): query head h reads kv head h / (H/Hkv); keys j with
// max(0, pos-window+1) <= j <= pos (window 0: from 0); scores scaled, softmax with running
// maximum, all in float.  One workgroup of 128 threads per (head, token); keys in chunks of
// 128, one key per thread for the scores, one output element per thread for the values.
#define AG_THREADS 128
#define AG_MAX_PER_THREAD 4            // head_dim <= 512
template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
        const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, T* __restrict__ out, int H, int Hkv,
        int hd, float scale, int window) {
    extern __shared__ float shared[];
    float* qs = shared;                 // [hd]
    float* sc = shared + hd;            // [AG_THREADS]
    float* scratch = sc + AG_THREADS;   // [16]
    const int n = blockIdx.x, h = blockIdx.y;     // tokens in x: a step may bring millions
    const int g = h / (H / Hkv);
    const int pos = tok_pos[n];
    const int* pages = table + (size_t)tok_seq[n] * table_stride;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const T* qrow = q + ((size_t)n * H + h) * hd;
    for (int d = threadIdx.x; d < hd; d += AG_THREADS) qs[d] = load_as_float(qrow + d);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[AG_MAX_PER_THREAD];
#pragma unroll
    for (int i = 0; i < AG_MAX_PER_THREAD; ++i) acc[i] = 0.f;

    for (int base = lo; base <= pos; base += AG_THREADS) {
        const int j = base + threadIdx.x;
        float s = -INFINITY;
        if (j <= pos) {
            const T* kr = k_pages + cache_region(pages[j / GFA_PAGE], g, Hkv, hd);
            float dot = 0.f;
            for (int d = 0; d < hd; ++d)
                dot = fmaf(qs[d], load_as_float(kr + key_offset(j % GFA_PAGE, d, hd)), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, block_max(s, scratch));
        const float alpha = expf(m - m_new);          // 0 on the first chunk (m = -inf)
        const float p = (j <= pos) ? expf(s - m_new) : 0.f;
        sc[threadIdx.x] = p;
        l = l * alpha + block_sum(p, scratch);        // contains the barrier that publishes sc
        const int count = (pos - base + 1 < AG_THREADS) ? pos - base + 1 : AG_THREADS;
#pragma unroll
        for (int i = 0; i < AG_MAX_PER_THREAD; ++i) {
            const int d = threadIdx.x + i * AG_THREADS;
            if (d < hd) {
                float a = acc[i] * alpha;
                for (int jj = 0; jj < count; ++jj) {
                    const int key = base + jj;
                    const T* vr = v_pages + value_elem(pages[key / GFA_PAGE], g, d,
                                                       key % GFA_PAGE, Hkv, hd);
                    a = fmaf(sc[jj], load_as_float(vr), a);
                }
                acc[i] = a;
            }
        }
        m = m_new;
        __syncthreads();
    }
    T* orow = out + ((size_t)n * H + h) * hd;
#pragma unroll
    for (int i = 0; i < AG_MAX_PER_THREAD; ++i) {
        const int d = threadIdx.x + i * AG_THREADS;
        if (d < hd) store_from_float(orow + d, acc[i] / l);
    }
}

extern "C" int gfa_attention_generic(const void* q, const void* k_pages, const void* v_pages,
                                     const int* tok_seq, const int* tok_pos, const int* table,
                                     int table_stride, void* out, int n_tokens, int H, int Hkv,
                                     int hd, float scale, int window, int is_bf16,
                                     hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (hd > AG_THREADS * AG_MAX_PER_THREAD || H > 65535) return (int)hipErrorInvalidValue;
    dim3 grid(n_tokens, H);
    const size_t shmem = (size_t)(hd + AG_THREADS + 16) * sizeof(float);
    if (is_bf16)
        attention_generic_kernel<bf16_t><<<grid, AG_THREADS, shmem, stream>>>(
            (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, tok_seq, tok_pos,
            table, table_stride, (bf16_t*)out, H, Hkv, hd, scale, window);
    else
        attention_generic_kernel<float><<<grid, AG_THREADS, shmem, stream>>>(
            (const float*)q, (const float*)k_pages, (const float*)v_pages, tok_seq, tok_pos,
            table, table_stride, (float*)out, H, Hkv, hd, scale, window);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// gate: out[n, i] = act(gu[n, i]) * gu[n, I + i]; act 0 = silu (model.py:227), 1 = the tanh
// form of gelu, 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
template <int ACT>
__device__ __forceinline__ float gate_act(float a) {
    if (ACT == 0) return a / (1.f + expf(-a));
    return 0.5f * a * (1.f + tanhf(0.7978845608028654f * (a + 0.044715f * a * a * a)));
}

template <typename T, int ACT>
__global__ void gate_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I,
                                size_t total) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x) {
        const size_t n = e / I;
        const int i = (int)(e % I);
        const float a = load_as_float(gu + n * 2 * I + i);
        const float b = load_as_float(gu + n * 2 * I + I + i);
        store_from_float(out + e, gate_act<ACT>(a) * b);
    }
}

// bfloat16 rows whose width is a multiple of 8: eight elements per thread, 16-byte accesses
template <int ACT>
__global__ __launch_bounds__(256) void gate_mul_bf16x8_kernel(const bf16_t* __restrict__ gu,
                                                              bf16_t* __restrict__ out, int I8,
                                                              size_t total8) {
    const size_t e = blockIdx.x * (size_t)256 + threadIdx.x;
    if (e >= total8) return;
    const size_t n = e / I8;
    const int i = (int)(e - n * I8);
    const uint4 a = ((const uint4*)gu)[n * 2 * I8 + i], b = ((const uint4*)gu)[n * 2 * I8 + I8 + i];
    const bf16_t* ae = (const bf16_t*)&a;
    const bf16_t* be = (const bf16_t*)&b;
    uint4 o;
    bf16_t* oe = (bf16_t*)&o;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        oe[j] = float_to_bf16(gate_act<ACT>(bf16_to_float(ae[j])) * bf16_to_float(be[j]));
    ((uint4*)out)[e] = o;
}

template <int ACT>
static int launch_gate_mul(const void* gu, void* out, int n_rows, int I, int is_bf16,
                           hipStream_t stream) {
    const size_t total = (size_t)n_rows * I;
    if (total == 0) return 0;
    if (is_bf16 && I % 8 == 0) {
        const size_t total8 = total / 8;
        gate_mul_bf16x8_kernel<ACT><<<(unsigned)((total8 + 255) / 256), 256, 0, stream>>>(
            (const bf16_t*)gu, (bf16_t*)out, I / 8, total8);
        return GFA_LAUNCH_RESULT();
    }
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (is_bf16)
        gate_mul_kernel<bf16_t, ACT><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total);
    else
        gate_mul_kernel<float, ACT><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, I, total);
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_gate_mul(const void* gu, void* out, int n_rows, int I, int act, int is_bf16,
                            hipStream_t stream) {
    if (act == 0) return launch_gate_mul<0>(gu, out, n_rows, I, is_bf16, stream);
    if (act == 1) return launch_gate_mul<1>(gu, out, n_rows, I, is_bf16, stream);
    return (int)hipErrorInvalidValue;
}

extern "C" int gfa_silu_mul(const void* gu, void* out, int n_rows, int I, int is_bf16,
                            hipStream_t stream) {
    return launch_gate_mul<0>(gu, out, n_rows, I, is_bf16, stream);
}

// --------------------------------------------------------------------------------------
// residual sum in float: res[e] += float(y[e])          (model.py:162-163)
template <typename T>
__global__ void add_into_kernel(float* __restrict__ res, const T* __restrict__ y, size_t total) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x)
        res[e] += load_as_float(y + e);
}

// bfloat16 addend, four elements per thread
__global__ __launch_bounds__(256) void add_into_bf16x4_kernel(float4* __restrict__ res,
                                                              const uint2* __restrict__ y,
                                                              size_t total4) {
    const size_t e = blockIdx.x * (size_t)256 + threadIdx.x;
    if (e >= total4) return;
    float4 r = res[e];
    const uint2 v = y[e];
    r.x += __uint_as_float(v.x << 16);
    r.y += __uint_as_float(v.x & 0xffff0000u);
    r.z += __uint_as_float(v.y << 16);
    r.w += __uint_as_float(v.y & 0xffff0000u);
    res[e] = r;
}

extern "C" int gfa_add_into(float* res, const void* y, size_t total, int y_bf16,
                            hipStream_t stream) {
    if (total == 0) return 0;
    if (y_bf16 && total % 4 == 0 && ((uintptr_t)res % 16 == 0) && ((uintptr_t)y % 8 == 0)) {
        const size_t total4 = total / 4;
        add_into_bf16x4_kernel<<<(unsigned)((total4 + 255) / 256), 256, 0, stream>>>(
            (float4*)res, (const uint2*)y, total4);
        return GFA_LAUNCH_RESULT();
    }
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (y_bf16)
        add_into_kernel<bf16_t><<<blocks, 256, 0, stream>>>(res, (const bf16_t*)y, total);
    else
        add_into_kernel<float><<<blocks, 256, 0, stream>>>(res, (const float*)y, total);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// x[e] = scale * x[e], then, if cap > 0, cap * tanh(x[e] / cap): a factor on the embedded
// rows or on the logits, and a soft cap of the logits, for plans that state one.
__global__ void scale_cap_kernel(float* __restrict__ x, size_t total, float scale, float cap) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x) {
        float v = x[e] * scale;
        if (cap > 0.f) v = cap * tanhf(v / cap);
        x[e] = v;
    }
}

extern "C" int gfa_scale_cap(float* x, size_t total, float scale, float cap, hipStream_t stream) {
    if (total == 0) return 0;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    scale_cap_kernel<<<blocks, 256, 0, stream>>>(x, total, scale, cap);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// naive matrix product with bfloat16 operands and float accumulation, one thread per
// output: the plain counterpart of the fast bfloat16 kernels (tests only).
__global__ void gemm_bf16_naive_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                       float* __restrict__ out, int M, int N, int K) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x, m = blockIdx.y;
    if (n >= N || m >= M) return;
    float acc = 0.f;
    for (int k = 0; k < K; ++k)
        acc = fmaf(bf16_to_float(a[(size_t)m * K + k]), bf16_to_float(w[(size_t)n * K + k]), acc);
    out[(size_t)m * N + n] = acc;
}

extern "C" int gfa_gemm_bf16_naive(const void* a, const void* w, float* out, int M, int N, int K,
                                   hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 65535) return (int)hipErrorInvalidValue;     // rows ride in the grid's second dimension
    dim3 grid((N + 255) / 256, M);
    gemm_bf16_naive_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)w, out, M, N, K);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// A sublayer's result joins the stream through a norm of its own ("sandwich" blocks):
//     res[r, :] += y[r, :] * rsqrt(mean(y[r, :]^2) + eps_y) * wy[:]
// and, if next_w is given, the norm that reads the stream next in the same pass:
//     out[r, :] = res[r, :] * rsqrt(mean(res[r, :]^2) + eps_n) * next_w[:]     (type T)
// y is float (a product's float sums).  One workgroup per row; statistics in float.
template <typename T>
__global__ __launch_bounds__(256) void normed_add_kernel(
        float* __restrict__ res, const float* __restrict__ y, const float* __restrict__ wy,
        float eps_y, const float* __restrict__ next_w, float eps_n, T* __restrict__ out, int dim) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * dim;
    const float* yr = y + row;
    float* rr = res + row;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) ss = fmaf(yr[d], yr[d], ss);
    ss = block_sum(ss, scratch);
    const float ry = rsqrtf(ss / (float)dim + eps_y);
    float sn = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {
        const float v = rr[d] + yr[d] * ry * wy[d];
        rr[d] = v;
        sn = fmaf(v, v, sn);
    }
    if (next_w == nullptr) return;
    sn = block_sum(sn, scratch);
    const float rn = rsqrtf(sn / (float)dim + eps_n);
    T* o = out + row;
    // every thread reads back only what it wrote itself
    for (int d = threadIdx.x; d < dim; d += 256) store_from_float(o + d, rr[d] * rn * next_w[d]);
}

// The same for rows of up to 1024 * VPT * 4 elements (a multiple of 4): y and the stream are
// read once with 16-byte loads and kept in registers between the sums and the stores.
template <typename T, int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void normed_add_vec_kernel(
        float* __restrict__ res, const float* __restrict__ y, const float* __restrict__ wy,
        float eps_y, const float* __restrict__ next_w, float eps_n, T* __restrict__ out, int dim) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * dim;
    const float4* y4 = (const float4*)(y + row);
    float4* r4 = (float4*)(res + row);
    const float4* wy4 = (const float4*)wy;
    const int n4 = dim >> 2;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 yv[VPT], rv[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        yv[j] = idx < n4 ? y4[idx] : zero;
        rv[j] = idx < n4 ? r4[idx] : zero;
        ss = fmaf(yv[j].x, yv[j].x, ss);
        ss = fmaf(yv[j].y, yv[j].y, ss);
        ss = fmaf(yv[j].z, yv[j].z, ss);
        ss = fmaf(yv[j].w, yv[j].w, ss);
    }
    ss = block_sum(ss, scratch);
    const float ry = rsqrtf(ss / (float)dim + eps_y);
    float sn = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = wy4[idx];
            rv[j].x += yv[j].x * ry * g.x;
            rv[j].y += yv[j].y * ry * g.y;
            rv[j].z += yv[j].z * ry * g.z;
            rv[j].w += yv[j].w * ry * g.w;
            r4[idx] = rv[j];
            sn = fmaf(rv[j].x, rv[j].x, sn);
            sn = fmaf(rv[j].y, rv[j].y, sn);
            sn = fmaf(rv[j].z, rv[j].z, sn);
            sn = fmaf(rv[j].w, rv[j].w, sn);
        }
    }
    if (next_w == nullptr) return;
    sn = block_sum(sn, scratch);
    const float rn = rsqrtf(sn / (float)dim + eps_n);
    const float4* nw4 = (const float4*)next_w;
    T* o = out + row;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = nw4[idx];
            store_from_float(o + 4 * idx + 0, rv[j].x * rn * g.x);
            store_from_float(o + 4 * idx + 1, rv[j].y * rn * g.y);
            store_from_float(o + 4 * idx + 2, rv[j].z * rn * g.z);
            store_from_float(o + 4 * idx + 3, rv[j].w * rn * g.w);
        }
    }
}

template <typename T>
static int launch_normed_add(float* res, const float* y, const float* wy, float eps_y,
                             const float* next_w, float eps_n, T* out, int n_rows, int dim,
                             hipStream_t stream) {
    if (dim % 4 == 0 && dim <= 8192) {
        if (dim <= 1024)
            normed_add_vec_kernel<T, 1, 256><<<n_rows, 256, 0, stream>>>(res, y, wy, eps_y, next_w, eps_n, out, dim);
        else if (dim <= 4096)
            normed_add_vec_kernel<T, 1, 1024><<<n_rows, 1024, 0, stream>>>(res, y, wy, eps_y, next_w, eps_n, out, dim);
        else
            normed_add_vec_kernel<T, 2, 1024><<<n_rows, 1024, 0, stream>>>(res, y, wy, eps_y, next_w, eps_n, out, dim);
    } else {
        normed_add_kernel<T><<<n_rows, 256, 0, stream>>>(res, y, wy, eps_y, next_w, eps_n, out, dim);
    }
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_normed_add(float* res, const float* y, const float* wy, float eps_y,
                              const float* next_w, float eps_n, void* out, int out_bf16,
                              int n_rows, int dim, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (out_bf16)
        return launch_normed_add<bf16_t>(res, y, wy, eps_y, next_w, eps_n, (bf16_t*)out, n_rows, dim, stream);
    return launch_normed_add<float>(res, y, wy, eps_y, next_w, eps_n, (float*)out, n_rows, dim, stream);
}

// --------------------------------------------------------------------------------------
// Activations of a feed-forward without a gate, element by element, in float:
//   0 silu, 1 gelu (tanh form), 3 gelu (exact, with erf), 2 xIELU with two numbers a = softplus(p), b = 1/2 + softplus(q):
//     z > 0: a z^2 + z/2        z <= 0: b (exp(z) - 1 - z) + z/2
template <int ACT>
__device__ __forceinline__ float activation(float z, float a, float b) {
    if (ACT == 0) return z / (1.f + expf(-z));
    if (ACT == 1) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    if (ACT == 3) return 0.5f * z * (1.f + erff(z * 0.7071067811865476f));
    return z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z);
}

template <typename T, int ACT>
__global__ void activate_kernel(const T* __restrict__ x, T* __restrict__ out, size_t total,
                                float a, float b) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x)
        store_from_float(out + e, activation<ACT>(load_as_float(x + e), a, b));
}

// eight bfloat16 per thread
template <int ACT>
__global__ __launch_bounds__(256) void activate_bf16x8_kernel(const uint4* __restrict__ x,
                                                              uint4* __restrict__ out, size_t total8,
                                                              float a, float b) {
    for (size_t e = blockIdx.x * (size_t)256 + threadIdx.x; e < total8; e += (size_t)gridDim.x * 256) {
        uint4 v = x[e];
        uint32_t* w = (uint32_t*)&v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = activation<ACT>(__uint_as_float(w[i] << 16), a, b);
            const float hi = activation<ACT>(__uint_as_float(w[i] & 0xffff0000u), a, b);
            w[i] = (uint32_t)float_to_bf16(lo) | ((uint32_t)float_to_bf16(hi) << 16);
        }
        out[e] = v;
    }
}

template <int ACT>
static int launch_activate(const void* x, void* out, size_t total, float a, float b, int is_bf16,
                           hipStream_t stream) {
    if (is_bf16 && total % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        const size_t n8 = total / 8;
        const int blocks = (int)((n8 + 255) / 256 < 262144 ? (n8 + 255) / 256 : 262144);
        activate_bf16x8_kernel<ACT><<<blocks, 256, 0, stream>>>((const uint4*)x, (uint4*)out, n8, a, b);
        return GFA_LAUNCH_RESULT();
    }
    const int blocks = (int)((total + 255) / 256 < 262144 ? (total + 255) / 256 : 262144);
    if (is_bf16)
        activate_kernel<bf16_t, ACT><<<blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, total, a, b);
    else
        activate_kernel<float, ACT><<<blocks, 256, 0, stream>>>((const float*)x, (float*)out, total, a, b);
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_activate(const void* x, void* out, size_t total, int act, float a, float b,
                            int is_bf16, hipStream_t stream) {
    if (total == 0) return 0;
    if (act == 0) return launch_activate<0>(x, out, total, a, b, is_bf16, stream);
    if (act == 1) return launch_activate<1>(x, out, total, a, b, is_bf16, stream);
    if (act == 2) return launch_activate<2>(x, out, total, a, b, is_bf16, stream);
    if (act == 3) return launch_activate<3>(x, out, total, a, b, is_bf16, stream);
    return (int)hipErrorInvalidValue;
}

// --------------------------------------------------------------------------------------
// out[r, :] = [a[r, :], b[r, :]] in type T from two float matrices of dim columns each: the
// operand of a product over the stream and the embedded rows side by side.
template <typename T>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                   T* __restrict__ out, int dim) {
    const size_t r = blockIdx.x;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        store_from_float(out + r * 2 * dim + d, a[r * dim + d]);
        store_from_float(out + r * 2 * dim + dim + d, b[r * dim + d]);
    }
}

extern "C" int gfa_concat_rows(const float* a, const float* b, void* out, int out_bf16, int n_rows,
                               int dim, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (out_bf16) concat_rows_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(a, b, (bf16_t*)out, dim);
    else concat_rows_kernel<float><<<n_rows, 256, 0, stream>>>(a, b, (float*)out, dim);
    return GFA_LAUNCH_RESULT();
}

// res[r, :] += bias[:]
__global__ void add_bias_kernel(float* __restrict__ res, const float* __restrict__ bias, int dim) {
    const size_t r = blockIdx.x;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) res[r * dim + d] += bias[d];
}

extern "C" int gfa_add_bias(float* res, const float* bias, int n_rows, int dim, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    add_bias_kernel<<<n_rows, 256, 0, stream>>>(res, bias, dim);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// A batch of float32 products with strides: for every b < B
//     out[b][m, n] = sum_k a[b][m, k] * w[b][n, k]
// with element (m, k) of a[b] at a + b sab + m sam + k (unit stride along k), element (n, k)
// of w[b] at w + b swb + n swn + k swk, element (m, n) of out[b] at out + b sob + m som + n.
// The same tiles and the same chain of fused multiply-adds per output as gemm_f32_kernel.
__global__ __launch_bounds__(256) void gemm_f32_strided_kernel(
        const float* __restrict__ a, const float* __restrict__ w, float* __restrict__ out,
        int M, int N, int K, long long sab, long long sam, long long swb, long long swn,
        long long swk, long long sob, long long som) {
    __shared__ float As[GF_BK][GF_BM + 4];
    __shared__ float Ws[GF_BK][GF_BN + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
    a += (size_t)blockIdx.z * sab;
    w += (size_t)blockIdx.z * swb;
    out += (size_t)blockIdx.z * sob;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += GF_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = threadIdx.x + i * 256;
            const int r = e >> 4, c = e & 15;
            const int k = k0 + c;
            const int m = m0 + r, n = n0 + r;
            As[c][r] = (m < M && k < K) ? a[(size_t)m * sam + k] : 0.f;
            Ws[c][r] = (n < N && k < K) ? w[(size_t)n * swn + (size_t)k * swk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GF_BK; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) out[(size_t)m * som + n] = acc[i][j];
        }
    }
}

extern "C" int gfa_gemm_f32_strided(const float* a, const float* w, float* out, int B, int M, int N,
                                    int K, long long sab, long long sam, long long swb,
                                    long long swn, long long swk, long long sob, long long som,
                                    hipStream_t stream) {
    if (B <= 0 || M <= 0 || N <= 0) return 0;
    if (B > 65535 || (M + GF_BM - 1) / GF_BM > 65535) return (int)hipErrorInvalidValue;
    dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM, B);
    gemm_f32_strided_kernel<<<grid, 256, 0, stream>>>(a, w, out, M, N, K, sab, sam, swb, swn, swk,
                                                      sob, som);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// out[n, :] += float(table[idx[n], :]): rows of a table picked by an index per token, added to
// the embedded rows (a learned position vector: idx = the tokens' positions).
template <typename T>
__global__ void add_table_rows_kernel(const T* __restrict__ table, const int* __restrict__ idx,
                                      float* __restrict__ out, int dim) {
    const int n = blockIdx.x;
    const T* row = table + (size_t)idx[n] * dim;
    float* o = out + (size_t)n * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] += load_as_float(row + d);
}

extern "C" int gfa_add_table_rows(const void* table, int table_bf16, const int* idx, float* out,
                                  int n_tokens, int dim, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (table_bf16)
        add_table_rows_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)table, idx, out, dim);
    else
        add_table_rows_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, idx, out, dim);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The embedding of the pair (previous token, token): out[n, :] += table[row(n), :] with
//   row = (previous * mul_prev + token * mul_cur) mod buckets       (64-bit integers)
//   row = buckets (the table's last row) for a sequence's first token.
// The previous token of the first token a step brings to a sequence is last[slot], where the
// step before left it; the workgroup of that first token reads it and then puts the
// sequence's last token of this step there (no other workgroup touches the entry).
template <typename T>
__global__ void pair_embed_add_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                                      const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                      const int* __restrict__ q_start, const int* __restrict__ slots,
                                      int* __restrict__ last, float* __restrict__ out, int dim,
                                      long long buckets, long long mul_prev, long long mul_cur) {
    const int n = blockIdx.x;
    const int b = tok_seq[n];
    const bool first_of_step = n == q_start[b];
    const int slot = slots[b];
    long long row = buckets;
    if (tok_pos[n] > 0) {
        const long long prev = first_of_step ? last[slot] : tokens[n - 1];
        row = (prev * mul_prev + (long long)tokens[n] * mul_cur) % buckets;
    }
    __syncthreads();                                   // every thread has read last[slot]
    if (first_of_step && threadIdx.x == 0) last[slot] = tokens[q_start[b + 1] - 1];
    const T* src = table + (size_t)row * dim;
    float* o = out + (size_t)n * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) o[d] += load_as_float(src + d);
}

extern "C" int gfa_pair_embed_add(const void* table, int table_bf16, const int* tokens,
                                  const int* tok_seq, const int* tok_pos, const int* q_start,
                                  const int* slots, int* last, float* out, int n_tokens, int dim,
                                  long long buckets, long long mul_prev, long long mul_cur,
                                  hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (buckets <= 0) return (int)hipErrorInvalidValue;
    if (table_bf16)
        pair_embed_add_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(
            (const bf16_t*)table, tokens, tok_seq, tok_pos, q_start, slots, last, out, dim, buckets,
            mul_prev, mul_cur);
    else
        pair_embed_add_kernel<float><<<n_tokens, 256, 0, stream>>>(
            (const float*)table, tokens, tok_seq, tok_pos, q_start, slots, last, out, dim, buckets,
            mul_prev, mul_cur);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// out[i, :] = T(x[r, :]), r = rows ? rows[i] : i: the float rows of the stream in the compute
// type, for a sublayer that reads the stream itself.
template <typename T>
__global__ void cast_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                 T* __restrict__ out, int dim) {
    const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
    const float* src = x + r * dim;
    T* o = out + (size_t)blockIdx.x * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) store_from_float(o + d, src[d]);
}

extern "C" int gfa_cast_rows(const float* x, const int* rows, void* out, int out_bf16, int n_rows,
                             int dim, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (out_bf16)
        cast_rows_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, rows, (bf16_t*)out, dim);
    else
        cast_rows_kernel<float><<<n_rows, 256, 0, stream>>>(x, rows, (float*)out, dim);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// A sublayer's result joins the stream through a gate and a norm of its own:
//   y'  = y * sigmoid(gate + gate_bias)          (gate: float sums of a projection, row stride
//                                                 gate_stride; gate null: y' = y)
//   res += y' * rsqrt(mean(y'^2) + eps_y) * wy
// and, from the same pass, what reads the stream next: next_mode 1: the RMS norm of the new
// rows with next_w and eps_n; 2: the new rows as they are; both in type T.  One workgroup per
// row of up to 256 * GN_MAX elements kept in registers; longer rows take the plain loops.
#define GN_MAX 32
template <typename T>
__global__ __launch_bounds__(256) void gated_normed_add_kernel(
        float* __restrict__ res, const float* __restrict__ y, const float* __restrict__ gate,
        long long gate_stride, const float* __restrict__ gate_bias, const float* __restrict__ wy,
        float eps_y, int next_mode, const float* __restrict__ next_w, float eps_n,
        T* __restrict__ out, int dim) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * dim;
    const float* yr = y + row;
    const float* gr = gate ? gate + (size_t)blockIdx.x * gate_stride : nullptr;
    float* rr = res + row;
    const bool fits = dim <= 256 * GN_MAX;
    float held[GN_MAX];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < GN_MAX; ++j) {
        const int d = threadIdx.x + 256 * j;
        float v = 0.f;
        if (fits && d < dim) {
            v = yr[d];
            if (gr) v *= 1.f / (1.f + expf(-(gr[d] + (gate_bias ? gate_bias[d] : 0.f))));
        }
        held[j] = v;
        ss = fmaf(v, v, ss);
    }
    if (!fits) {
        for (int d = threadIdx.x; d < dim; d += 256) {
            float v = yr[d];
            if (gr) v *= 1.f / (1.f + expf(-(gr[d] + (gate_bias ? gate_bias[d] : 0.f))));
            ss = fmaf(v, v, ss);
        }
    }
    ss = block_sum(ss, scratch);
    const float ry = rsqrtf(ss / (float)dim + eps_y);
    float sn = 0.f;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            if (d < dim) {
                const float v = rr[d] + held[j] * ry * wy[d];
                rr[d] = v;
                held[j] = v;
                sn = fmaf(v, v, sn);
            }
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) {
            float v = yr[d];
            if (gr) v *= 1.f / (1.f + expf(-(gr[d] + (gate_bias ? gate_bias[d] : 0.f))));
            v = rr[d] + v * ry * wy[d];
            rr[d] = v;
            sn = fmaf(v, v, sn);
        }
    }
    if (next_mode == 0) return;
    float rn = 1.f;
    if (next_mode == 1) {
        sn = block_sum(sn, scratch);
        rn = rsqrtf(sn / (float)dim + eps_n);
    }
    T* o = out + row;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            if (d < dim) store_from_float(o + d, next_mode == 1 ? held[j] * rn * next_w[d] : held[j]);
        }
    } else {
        // every thread reads back only what it wrote itself
        for (int d = threadIdx.x; d < dim; d += 256)
            store_from_float(o + d, next_mode == 1 ? rr[d] * rn * next_w[d] : rr[d]);
    }
}

// The same for rows of up to 1024 * VPT * 4 elements (a multiple of 4, gate rows at addresses
// that are multiples of 16): everything is read once with 16-byte loads and kept in registers
// between the sums and the stores.
template <typename T, int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void gated_normed_add_vec_kernel(
        float* __restrict__ res, const float* __restrict__ y, const float* __restrict__ gate,
        long long gate_stride, const float* __restrict__ gate_bias, const float* __restrict__ wy,
        float eps_y, int next_mode, const float* __restrict__ next_w, float eps_n,
        T* __restrict__ out, int dim) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * dim;
    const float4* y4 = (const float4*)(y + row);
    const float4* g4 = gate ? (const float4*)(gate + (size_t)blockIdx.x * gate_stride) : nullptr;
    const float4* b4 = (const float4*)gate_bias;
    float4* r4 = (float4*)(res + row);
    const float4* wy4 = (const float4*)wy;
    const int n4 = dim >> 2;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 yv[VPT], rv[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        const bool in = idx < n4;
        yv[j] = in ? y4[idx] : zero;
        rv[j] = in ? r4[idx] : zero;
        if (g4 && in) {
            float4 g = g4[idx];
            if (b4) {
                const float4 b = b4[idx];
                g.x += b.x; g.y += b.y; g.z += b.z; g.w += b.w;
            }
            yv[j].x *= 1.f / (1.f + expf(-g.x));
            yv[j].y *= 1.f / (1.f + expf(-g.y));
            yv[j].z *= 1.f / (1.f + expf(-g.z));
            yv[j].w *= 1.f / (1.f + expf(-g.w));
        }
        ss = fmaf(yv[j].x, yv[j].x, ss);
        ss = fmaf(yv[j].y, yv[j].y, ss);
        ss = fmaf(yv[j].z, yv[j].z, ss);
        ss = fmaf(yv[j].w, yv[j].w, ss);
    }
    ss = block_sum(ss, scratch);
    const float ry = rsqrtf(ss / (float)dim + eps_y);
    float sn = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = wy4[idx];
            rv[j].x += yv[j].x * ry * g.x;
            rv[j].y += yv[j].y * ry * g.y;
            rv[j].z += yv[j].z * ry * g.z;
            rv[j].w += yv[j].w * ry * g.w;
            r4[idx] = rv[j];
            sn = fmaf(rv[j].x, rv[j].x, sn);
            sn = fmaf(rv[j].y, rv[j].y, sn);
            sn = fmaf(rv[j].z, rv[j].z, sn);
            sn = fmaf(rv[j].w, rv[j].w, sn);
        }
    }
    if (next_mode == 0) return;
    float rn = 1.f;
    if (next_mode == 1) {
        sn = block_sum(sn, scratch);
        rn = rsqrtf(sn / (float)dim + eps_n);
    }
    const float4* nw4 = (const float4*)next_w;
    T* o = out + row;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            float4 v = rv[j];
            if (next_mode == 1) {
                const float4 g = nw4[idx];
                v.x *= rn * g.x; v.y *= rn * g.y; v.z *= rn * g.z; v.w *= rn * g.w;
            }
            store_from_float(o + 4 * idx + 0, v.x);
            store_from_float(o + 4 * idx + 1, v.y);
            store_from_float(o + 4 * idx + 2, v.z);
            store_from_float(o + 4 * idx + 3, v.w);
        }
    }
}

template <typename T>
static int launch_gated_normed_add(float* res, const float* y, const float* gate, long long gate_stride,
                                   const float* gate_bias, const float* wy, float eps_y, int next_mode,
                                   const float* next_w, float eps_n, T* out, int n_rows, int dim,
                                   hipStream_t stream) {
    const bool vec = dim % 4 == 0 && dim <= 8192 && (!gate || (gate_stride % 4 == 0 && (size_t)gate % 16 == 0))
        && (size_t)res % 16 == 0 && (size_t)y % 16 == 0 && (size_t)wy % 16 == 0
        && (size_t)gate_bias % 16 == 0 && (size_t)next_w % 16 == 0;
#define GFA_GN_ARGS res, y, gate, gate_stride, gate_bias, wy, eps_y, next_mode, next_w, eps_n, out, dim
    if (!vec)
        gated_normed_add_kernel<T><<<n_rows, 256, 0, stream>>>(GFA_GN_ARGS);
    else if (dim <= 1024)
        gated_normed_add_vec_kernel<T, 1, 256><<<n_rows, 256, 0, stream>>>(GFA_GN_ARGS);
    else if (dim <= 4096)
        gated_normed_add_vec_kernel<T, 1, 1024><<<n_rows, 1024, 0, stream>>>(GFA_GN_ARGS);
    else
        gated_normed_add_vec_kernel<T, 2, 1024><<<n_rows, 1024, 0, stream>>>(GFA_GN_ARGS);
#undef GFA_GN_ARGS
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_gated_normed_add(float* res, const float* y, const float* gate,
                                    long long gate_stride, const float* gate_bias, const float* wy,
                                    float eps_y, int next_mode, const float* next_w, float eps_n,
                                    void* out, int out_bf16, int n_rows, int dim,
                                    hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (next_mode < 0 || next_mode > 2 || (next_mode == 1 && !next_w) || (next_mode && !out))
        return (int)hipErrorInvalidValue;
    if (out_bf16)
        return launch_gated_normed_add<bf16_t>(res, y, gate, gate_stride, gate_bias, wy, eps_y, next_mode,
                                               next_w, eps_n, (bf16_t*)out, n_rows, dim, stream);
    return launch_gated_normed_add<float>(res, y, gate, gate_stride, gate_bias, wy, eps_y, next_mode,
                                          next_w, eps_n, (float*)out, n_rows, dim, stream);
}

// --------------------------------------------------------------------------------------
// Layer norm with a weight and no bias:
//   out[i, :] = (x[r, :] - mean) * rsqrt(mean((x[r, :] - mean)^2) + eps) * w[:],  r = rows ? rows[i] : i
// The variance is the mean of the squared deviations (a second pass over the row, which a
// thread keeps in registers up to 256 * GN_MAX elements).  Float arithmetic, one rounding at
// the store.
template <typename T>
__global__ __launch_bounds__(256) void layer_norm_kernel(
        const float* __restrict__ x, const float* __restrict__ w, const int* __restrict__ rows,
        T* __restrict__ out, int dim, float eps) {
    __shared__ float scratch[16];
    const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
    const float* xr = x + r * dim;
    const bool fits = dim <= 256 * GN_MAX;
    float held[GN_MAX];
    float sum = 0.f;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            held[j] = d < dim ? xr[d] : 0.f;
            sum += held[j];
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) sum += xr[d];
    }
    const float mean = block_sum(sum, scratch) / (float)dim;
    float sq = 0.f;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            const float c = d < dim ? held[j] - mean : 0.f;
            sq = fmaf(c, c, sq);
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float c = xr[d] - mean;
            sq = fmaf(c, c, sq);
        }
    }
    const float rs = rsqrtf(block_sum(sq, scratch) / (float)dim + eps);
    T* o = out + (size_t)blockIdx.x * dim;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            if (d < dim) store_from_float(o + d, (held[j] - mean) * rs * w[d]);
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) store_from_float(o + d, (xr[d] - mean) * rs * w[d]);
    }
}

extern "C" int gfa_layer_norm(const float* x, const float* w, const int* rows, void* out, int out_bf16,
                              int n_rows, int dim, float eps, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (out_bf16)
        layer_norm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, w, rows, (bf16_t*)out, dim, eps);
    else
        layer_norm_kernel<float><<<n_rows, 256, 0, stream>>>(x, w, rows, (float*)out, dim, eps);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// A sublayer's result joins a stream that is normed AFTER the sum:
//   y    = ya                                                   (yb null), or
//   y    = (ya rsqrt(mean(ya^2) + eps_b) wa + yb rsqrt(mean(yb^2) + eps_b) wb) / 2
//          (two branches that read the same input, each RMS-normed with a weight of its own)
//   v    = alpha * res + ls * y                                 (ls: a weight per column, or null)
//   res  = (v - mean(v)) * rsqrt(mean((v - mean(v))^2) + eps) * w
// and, from the same pass, the new rows in type T for whoever reads the stream next (out null:
// not).  One workgroup per row; a thread keeps its elements in registers up to 256 * GN_MAX
// per row, longer rows go through res (every thread reads back only what it wrote).
template <typename T>
__global__ __launch_bounds__(256) void post_norm_join_kernel(
        float* __restrict__ res, const float* __restrict__ ya, const float* __restrict__ yb,
        const float* __restrict__ wa, const float* __restrict__ wb, float eps_b,
        const float* __restrict__ ls, float alpha, const float* __restrict__ w, float eps,
        T* __restrict__ out, int dim) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * dim;
    float* rr = res + row;
    const float* ar = ya + row;
    const float* br = yb ? yb + row : nullptr;
    const bool fits = dim <= 256 * GN_MAX;
    float fa = 1.f, fb = 0.f;
    if (br) {
        float sa = 0.f, sb = 0.f;
        for (int d = threadIdx.x; d < dim; d += 256) {
            sa = fmaf(ar[d], ar[d], sa);
            sb = fmaf(br[d], br[d], sb);
        }
        fa = 0.5f * rsqrtf(block_sum(sa, scratch) / (float)dim + eps_b);
        fb = 0.5f * rsqrtf(block_sum(sb, scratch) / (float)dim + eps_b);
    }
    float held[GN_MAX];
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < GN_MAX; ++j) {
        const int d = threadIdx.x + 256 * j;
        float v = 0.f;
        if (fits && d < dim) {
            const float y = br ? ar[d] * fa * wa[d] + br[d] * fb * wb[d] : ar[d];
            v = fmaf(alpha, rr[d], ls ? ls[d] * y : y);
        }
        held[j] = v;
        sum += v;
    }
    if (!fits) {
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float y = br ? ar[d] * fa * wa[d] + br[d] * fb * wb[d] : ar[d];
            const float v = fmaf(alpha, rr[d], ls ? ls[d] * y : y);
            rr[d] = v;
            sum += v;
        }
    }
    const float mean = block_sum(sum, scratch) / (float)dim;
    float sq = 0.f;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            const float c = d < dim ? held[j] - mean : 0.f;
            sq = fmaf(c, c, sq);
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float c = rr[d] - mean;
            sq = fmaf(c, c, sq);
        }
    }
    const float rs = rsqrtf(block_sum(sq, scratch) / (float)dim + eps);
    T* o = out ? out + row : nullptr;
    if (fits) {
#pragma unroll
        for (int j = 0; j < GN_MAX; ++j) {
            const int d = threadIdx.x + 256 * j;
            if (d < dim) {
                const float v = (held[j] - mean) * rs * w[d];
                rr[d] = v;
                if (o) store_from_float(o + d, v);
            }
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float v = (rr[d] - mean) * rs * w[d];
            rr[d] = v;
            if (o) store_from_float(o + d, v);
        }
    }
}

// The same for rows of up to THREADS * VPT * 4 elements (a multiple of 4, every pointer at a
// multiple of 16 bytes): everything is read once with 16-byte loads and kept in registers
// between the sums and the stores.
template <typename T, int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void post_norm_join_vec_kernel(
        float* __restrict__ res, const float* __restrict__ ya, const float* __restrict__ yb,
        const float* __restrict__ wa, const float* __restrict__ wb, float eps_b,
        const float* __restrict__ ls, float alpha, const float* __restrict__ w, float eps,
        T* __restrict__ out, int dim) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * dim;
    float4* r4 = (float4*)(res + row);
    const float4* a4 = (const float4*)(ya + row);
    const float4* b4 = yb ? (const float4*)(yb + row) : nullptr;
    const int n4 = dim >> 2;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 v[VPT], yv[VPT], zv[VPT];
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        const bool in = idx < n4;
        v[j] = in ? r4[idx] : zero;
        yv[j] = in ? a4[idx] : zero;
        zv[j] = (in && b4) ? b4[idx] : zero;
        sa += yv[j].x * yv[j].x + yv[j].y * yv[j].y + yv[j].z * yv[j].z + yv[j].w * yv[j].w;
        sb += zv[j].x * zv[j].x + zv[j].y * zv[j].y + zv[j].z * zv[j].z + zv[j].w * zv[j].w;
    }
    float fa = 1.f, fb = 0.f;
    if (b4) {
        fa = 0.5f * rsqrtf(block_sum(sa, scratch) / (float)dim + eps_b);
        fb = 0.5f * rsqrtf(block_sum(sb, scratch) / (float)dim + eps_b);
    }
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            float4 y = yv[j];
            if (b4) {
                const float4 ga = ((const float4*)wa)[idx], gb = ((const float4*)wb)[idx];
                y.x = y.x * fa * ga.x + zv[j].x * fb * gb.x;
                y.y = y.y * fa * ga.y + zv[j].y * fb * gb.y;
                y.z = y.z * fa * ga.z + zv[j].z * fb * gb.z;
                y.w = y.w * fa * ga.w + zv[j].w * fb * gb.w;
            }
            if (ls) {
                const float4 l = ((const float4*)ls)[idx];
                y.x *= l.x; y.y *= l.y; y.z *= l.z; y.w *= l.w;
            }
            v[j].x = fmaf(alpha, v[j].x, y.x);
            v[j].y = fmaf(alpha, v[j].y, y.y);
            v[j].z = fmaf(alpha, v[j].z, y.z);
            v[j].w = fmaf(alpha, v[j].w, y.w);
            sum += v[j].x + v[j].y + v[j].z + v[j].w;
        }
    }
    const float mean = block_sum(sum, scratch) / (float)dim;
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            v[j].x -= mean; v[j].y -= mean; v[j].z -= mean; v[j].w -= mean;
            sq += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
        }
    }
    const float rs = rsqrtf(block_sum(sq, scratch) / (float)dim + eps);
    T* o = out ? out + row : nullptr;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int idx = threadIdx.x + j * THREADS;
        if (idx < n4) {
            const float4 g = ((const float4*)w)[idx];
            float4 x = v[j];
            x.x *= rs * g.x; x.y *= rs * g.y; x.z *= rs * g.z; x.w *= rs * g.w;
            r4[idx] = x;
            if (o) {
                store_from_float(o + 4 * idx + 0, x.x);
                store_from_float(o + 4 * idx + 1, x.y);
                store_from_float(o + 4 * idx + 2, x.z);
                store_from_float(o + 4 * idx + 3, x.w);
            }
        }
    }
}

template <typename T>
static int launch_post_norm_join(float* res, const float* ya, const float* yb, const float* wa,
                                 const float* wb, float eps_b, const float* ls, float alpha,
                                 const float* w, float eps, T* out, int n_rows, int dim,
                                 hipStream_t stream) {
    const bool vec = dim % 4 == 0 && dim <= 8192 && (size_t)res % 16 == 0 && (size_t)ya % 16 == 0
        && (size_t)yb % 16 == 0 && (size_t)wa % 16 == 0 && (size_t)wb % 16 == 0 && (size_t)ls % 16 == 0
        && (size_t)w % 16 == 0;
#define GFA_PJ_ARGS res, ya, yb, wa, wb, eps_b, ls, alpha, w, eps, out, dim
    if (!vec)
        post_norm_join_kernel<T><<<n_rows, 256, 0, stream>>>(GFA_PJ_ARGS);
    else if (dim <= 1024)
        post_norm_join_vec_kernel<T, 1, 256><<<n_rows, 256, 0, stream>>>(GFA_PJ_ARGS);
    else if (dim <= 4096)
        post_norm_join_vec_kernel<T, 1, 1024><<<n_rows, 1024, 0, stream>>>(GFA_PJ_ARGS);
    else
        post_norm_join_vec_kernel<T, 2, 1024><<<n_rows, 1024, 0, stream>>>(GFA_PJ_ARGS);
#undef GFA_PJ_ARGS
    return GFA_LAUNCH_RESULT();
}

extern "C" int gfa_post_norm_join(float* res, const float* ya, const float* yb, const float* wa,
                                  const float* wb, float eps_b, const float* ls, float alpha,
                                  const float* w, float eps, void* out, int out_bf16, int n_rows,
                                  int dim, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (!res || !ya || !w || (yb && (!wa || !wb))) return (int)hipErrorInvalidValue;
    if (out_bf16)
        return launch_post_norm_join<bf16_t>(res, ya, yb, wa, wb, eps_b, ls, alpha, w, eps, (bf16_t*)out,
                                             n_rows, dim, stream);
    return launch_post_norm_join<float>(res, ya, yb, wa, wb, eps_b, ls, alpha, w, eps, (float*)out,
                                        n_rows, dim, stream);
}

// --------------------------------------------------------------------------------------
// Rotation of heads that lie in float rows, in place: rows [N, row_width], H heads of hd
// elements from column `off`; the first `rot` elements of every head are turned by
// pos * freqs[i], pairs (2i, 2i + 1) (layout 0) or (i, i + rot / 2) (layout 1):
//   (u, v) -> (u c - v s, v c + u s),  c = trig * cos(a), s = trig * sin(a)
// and then EVERY element of the head is multiplied by `factor` - heads from number `late` on
// by `late_factor` instead (q and k that lie one behind the other, k with a factor of its
// own).  One thread per pair, or per element behind the rotated part; grid (tokens, heads).
__global__ void rotate_rows_kernel(float* __restrict__ x, int row_width, int off, int hd, int rot,
                                   int layout, const float* __restrict__ freqs, float trig,
                                   float factor, int late, float late_factor,
                                   const int* __restrict__ tok_pos) {
    const int n = blockIdx.x, h = blockIdx.y;
    float* head = x + (size_t)n * row_width + off + h * hd;
    const float pos = (float)tok_pos[n];
    const float f = h >= late ? late_factor : factor;
    const int half = rot >> 1;
    for (int e = threadIdx.x; e < half + (hd - rot); e += blockDim.x) {
        if (e < half) {
            const int iu = layout == 0 ? 2 * e : e, iv = layout == 0 ? 2 * e + 1 : e + half;
            float sn, cs;
            sincosf(pos * freqs[e], &sn, &cs);
            sn *= trig;
            cs *= trig;
            const float u = head[iu], v = head[iv];
            head[iu] = (u * cs - v * sn) * f;
            head[iv] = (v * cs + u * sn) * f;
        } else {
            head[rot + e - half] *= f;
        }
    }
}

extern "C" int gfa_rotate_rows(float* x, int row_width, int off, int n_heads, int hd, int rot,
                               int layout, const float* freqs, float trig, float factor, int late,
                               float late_factor, const int* tok_pos, int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0 || n_heads <= 0) return 0;
    if (rot < 0 || rot > hd || rot % 2 || (rot && !freqs) || n_heads > 65535 ||
            off + n_heads * hd > row_width)
        return (int)hipErrorInvalidValue;
    rotate_rows_kernel<<<dim3(n_tokens, n_heads), 64, 0, stream>>>(x, row_width, off, hd, rot, layout,
                                                                  freqs, trig, factor, late, late_factor,
                                                                  tok_pos);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The gate over float sums, rounded once: out[n, i] = act(gu[n, i]) * gu[n, I + i] as
// bfloat16, gu float [N, 2 I] (the sums of a product whose rows are the gate rows and then
// the up rows).  act 0: silu, 1: gelu (tanh form).
template <int ACT>
__global__ void gate_mul_sums_kernel(const float* __restrict__ gu, bf16_t* __restrict__ out, int I,
                                     size_t total) {
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total;
         e += (size_t)gridDim.x * blockDim.x) {
        const size_t n = e / I;
        const int i = (int)(e % I);
        out[e] = float_to_bf16(gate_act<ACT>(gu[n * 2 * I + i]) * gu[n * 2 * I + I + i]);
    }
}

extern "C" int gfa_gate_mul_sums(const float* gu, void* out, int n_rows, int I, int act,
                                 hipStream_t stream) {
    const size_t total = (size_t)n_rows * I;
    if (total == 0) return 0;
    const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    if (act == 0) gate_mul_sums_kernel<0><<<blocks, 256, 0, stream>>>(gu, (bf16_t*)out, I, total);
    else if (act == 1) gate_mul_sums_kernel<1><<<blocks, 256, 0, stream>>>(gu, (bf16_t*)out, I, total);
    else return (int)hipErrorInvalidValue;
    return GFA_LAUNCH_RESULT();
}

// y[n, :] *= sigmoid(g[n * g_stride]): a gate of one number per row on float rows.
__global__ void scale_rows_sigmoid_kernel(float* __restrict__ y, const float* __restrict__ g,
                                          long long g_stride, int dim) {
    const float f = 1.f / (1.f + expf(-g[(size_t)blockIdx.x * g_stride]));
    float* row = y + (size_t)blockIdx.x * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) row[d] *= f;
}

extern "C" int gfa_scale_rows_sigmoid(float* y, const float* g, long long g_stride, int n_rows, int dim,
                                      hipStream_t stream) {
    if (n_rows <= 0) return 0;
    scale_rows_sigmoid_kernel<<<n_rows, 256, 0, stream>>>(y, g, g_stride, dim);
    return GFA_LAUNCH_RESULT();
}
