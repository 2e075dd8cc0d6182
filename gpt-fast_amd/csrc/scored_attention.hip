// Attention over the paged cache whose scores take further steps between the dot product and
// the softmax, and whose keys and values may have different sizes; all arithmetic in float.
//
// For the token at position i of a sequence, head h (kv head g = h / (H / G)) and key j with
// max(0, i - window + 1) <= j <= i (window 0: from 0):
//     s_h(j) = (q_h . k_g(j)) * scale * temperature[h]                  (temperature optional)
//     s_h(j) = softcap * tanh(s_h(j) / softcap)                         (softcap > 0)
//     s_h(j) = s_h(j) + bias[row(i - j), h]                             (bias optional)
//     s_h(j) = s_h(j) - r1[h] ln(1 + r2[h] (i - j))                     (r1, r2 optional)
//     z_h(j) = sum_h' talk[h, h'] s_h'(j)                               (talk optional)
//     out_h  = sum_j softmax_j(z_h)(j) v_g(j)
// With a sink the softmax's denominator has one more term, exp(0): a key of score zero that
// carries no value (the running maximum starts at 0 and the running sum at 1).
// row(n) = lookup[n] for n < n_lookup, else bias_rows - 1 (the host fills the lookup table).
//
// The cache keeps keys and values in the orders of common.h (key_offset, value_offset) with
// head sizes hd for keys and vd for values.  q and out are addressed by strides, so rows may
// lie token by token or head by head.
//
// Also here: the kernels that make q, keys and values of two mixers from their projections'
// float sums and put keys and values into the cache (unit-norm heads with biases; a normed
// latent with one rotated key part).
#include "common.h"

#define SA_THREADS 256
#define SA_WAVES 4

struct SAShape {
    int H, G, hd, vd;
    long long q_tok, q_head, o_tok, o_head;      // strides in elements
    int table_stride, window;
    float scale, softcap;
    int bias_rows, n_lookup;
    int sink;
};

template <typename T> struct Pack8;
template <> struct Pack8<bf16_t> {
    uint4 raw;
    __device__ __forceinline__ void load(const bf16_t* p) { raw = *(const uint4*)p; }
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = ((const uint32_t*)&raw)[i >> 1];
        return (i & 1) ? __uint_as_float(w & 0xffff0000u) : __uint_as_float(w << 16);
    }
};
template <> struct Pack8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const float* p) {
        a = *(const float4*)p;
        b = *(const float4*)(p + 4);
    }
    __device__ __forceinline__ float get(int i) const {
        return i < 4 ? ((const float*)&a)[i] : ((const float*)&b)[i - 4];
    }
};

// One workgroup per (token, block of 4 * HPW heads): wave w owns heads w, w + 4, ... of the
// block; a lane is a key of the page for the scores and a value element for the sums.  Keys
// are walked a page at a time, pages counted from the sequence's start, so a token's result
// does not depend on how its sequence was cut into steps.
template <typename T, int HPW, int VPT>
__global__ __launch_bounds__(SA_THREADS) void scored_attention_kernel(
        const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, const float* __restrict__ temperature,
        const float* __restrict__ bias, const int* __restrict__ lookup,
        const float* __restrict__ talk, const float* __restrict__ r1, const float* __restrict__ r2,
        T* __restrict__ out, SAShape s) {
    extern __shared__ __attribute__((aligned(16))) float sa_lds[];
    constexpr int HB = SA_WAVES * HPW;
    const int nh = s.H < HB ? s.H : HB;          // heads a block really has
    float* qs = sa_lds;                          // [nh][hd]
    float* sc = qs + nh * s.hd;                  // [HB][64] scores before the mix
    float* pr = sc + HB * GFA_PAGE;              // [HB][64] softmax weights
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x, h0 = blockIdx.y * HB;
    const int pos = tok_pos[n];
    const int* pages = table + (size_t)tok_seq[n] * s.table_stride;
    const int lo = (s.window > 0 && pos - s.window + 1 > 0) ? pos - s.window + 1 : 0;
    const int per_group = s.H / s.G;

    for (int e = threadIdx.x; e < nh * s.hd; e += SA_THREADS) {
        const int hl = e / s.hd, d = e - hl * s.hd;
        qs[e] = (h0 + hl < s.H)
            ? load_as_float(q + (size_t)n * s.q_tok + (size_t)(h0 + hl) * s.q_head + d) : 0.f;
    }
    float m[HPW], l[HPW], acc[HPW][VPT];
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        m[i] = s.sink ? 0.f : -INFINITY;
        l[i] = s.sink ? 1.f : 0.f;
#pragma unroll
        for (int e = 0; e < VPT; ++e) acc[i][e] = 0.f;
    }
    __syncthreads();

    for (int pg = lo / GFA_PAGE; pg <= pos / GFA_PAGE; ++pg) {
        const int page = pages[pg];
        const int j = pg * GFA_PAGE + lane;
        const bool seen = j >= lo && j <= pos;
        float z[HPW];
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int hl = wave + SA_WAVES * i, h = h0 + hl;
            z[i] = 0.f;
            if (h >= s.H || !seen) continue;
            const int g = h / per_group;
            const T* kr = k_pages + cache_region(page, g, s.G, s.hd);
            const float* qh = qs + hl * s.hd;
            float dot = 0.f;
            if (s.hd % 8 == 0) {
                for (int d = 0; d < s.hd; d += 8) {
                    Pack8<T> kk;
                    kk.load(kr + key_offset(lane, d, s.hd));
#pragma unroll
                    for (int t = 0; t < 8; ++t) dot = fmaf(qh[d + t], kk.get(t), dot);
                }
            } else {
                for (int d = 0; d < s.hd; ++d)
                    dot = fmaf(qh[d], load_as_float(kr + key_offset(lane, d, s.hd)), dot);
            }
            float v = dot * s.scale;
            if (temperature) v *= temperature[h];
            if (s.softcap > 0.f) v = s.softcap * tanhf(v / s.softcap);
            if (bias) {
                const int dist = pos - j;
                const int row = dist < s.n_lookup ? lookup[dist] : s.bias_rows - 1;
                v += bias[(size_t)row * s.H + h];
            }
            if (r1) v -= r1[h] * log1pf(r2[h] * (float)(pos - j));
            z[i] = v;
        }
        if (talk) {
#pragma unroll
            for (int i = 0; i < HPW; ++i) sc[(wave + SA_WAVES * i) * GFA_PAGE + lane] = z[i];
            __syncthreads();
#pragma unroll
            for (int i = 0; i < HPW; ++i) {
                const int h = wave + SA_WAVES * i;           // talk: one block holds every head
                if (h >= s.H) continue;
                float v = 0.f;
                for (int g = 0; g < s.H; ++g) v = fmaf(talk[h * s.H + g], sc[g * GFA_PAGE + lane], v);
                z[i] = v;
            }
        }
        float alpha[HPW];
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int hl = wave + SA_WAVES * i;
            const float v = seen ? z[i] : -INFINITY;
            const float m_new = fmaxf(m[i], wave_max(v));
            alpha[i] = m_new == -INFINITY ? 1.f : expf(m[i] - m_new);
            const float p = seen ? expf(v - m_new) : 0.f;
            l[i] = l[i] * alpha[i] + wave_sum(p);
            m[i] = m_new;
            pr[hl * GFA_PAGE + lane] = p;
        }
        __syncthreads();
        // keys of this page that are seen: [j_lo, j_hi], in groups of eight
        const int j_lo = lo > pg * GFA_PAGE ? lo - pg * GFA_PAGE : 0;
        const int j_hi = pos - pg * GFA_PAGE < GFA_PAGE - 1 ? pos - pg * GFA_PAGE : GFA_PAGE - 1;
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int hl = wave + SA_WAVES * i, h = h0 + hl;
            if (h >= s.H) continue;
            const int g = h / per_group;
            const T* vr = v_pages + cache_region(page, g, s.G, s.vd);
            const float* ph = pr + hl * GFA_PAGE;
#pragma unroll
            for (int e = 0; e < VPT; ++e) {
                const int d = lane + 64 * e;
                float a = acc[i][e] * alpha[i];
                if (d < s.vd) {
                    for (int kg = j_lo >> 3; kg <= j_hi >> 3; ++kg) {
                        Pack8<T> vv;
                        vv.load(vr + value_offset(d, kg * 8, s.vd));
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            const int key = kg * 8 + t;
                            // the pool is not cleared: what lies beyond the seen keys may be anything
                            const float val = (key >= j_lo && key <= j_hi) ? vv.get(t) : 0.f;
                            a = fmaf(ph[key], val, a);
                        }
                    }
                }
                acc[i][e] = a;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        const int h = h0 + wave + SA_WAVES * i;
        if (h >= s.H) continue;
        T* o = out + (size_t)n * s.o_tok + (size_t)h * s.o_head;
#pragma unroll
        for (int e = 0; e < VPT; ++e) {
            const int d = lane + 64 * e;
            if (d < s.vd) store_from_float(o + d, acc[i][e] / l[i]);
        }
    }
}

template <typename T, int HPW, int VPT>
static int sa_launch(const void* q, const void* k_pages, const void* v_pages, const int* tok_seq,
                     const int* tok_pos, const int* table, const float* temperature,
                     const float* bias, const int* lookup, const float* talk, const float* r1,
                     const float* r2, void* out, int n_tokens, const SAShape& s, hipStream_t stream) {
    constexpr int HB = SA_WAVES * HPW;
    const size_t shmem = ((size_t)(s.H < HB ? s.H : HB) * s.hd + (size_t)HB * 2 * GFA_PAGE) * sizeof(float);
    if (shmem > 160 * 1024) return (int)hipErrorInvalidValue;
    if (shmem > 64 * 1024) {
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute((const void*)scored_attention_kernel<T, HPW, VPT>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
    }
    dim3 grid(n_tokens, (s.H + HB - 1) / HB);
    scored_attention_kernel<T, HPW, VPT><<<grid, SA_THREADS, shmem, stream>>>(
        (const T*)q, (const T*)k_pages, (const T*)v_pages, tok_seq, tok_pos, table, temperature,
        bias, lookup, talk, r1, r2, (T*)out, s);
    return GFA_LAUNCH_RESULT();
}

template <typename T>
static int sa_dispatch(const void* q, const void* k_pages, const void* v_pages, const int* tok_seq,
                       const int* tok_pos, const int* table, const float* temperature,
                       const float* bias, const int* lookup, const float* talk, const float* r1,
                       const float* r2, void* out, int n_tokens, const SAShape& s, hipStream_t stream) {
    // heads per wave: with a mix one workgroup holds every head; without, one head per wave
    const int hpw = talk ? (s.H + SA_WAVES - 1) / SA_WAVES : 1;
    const int vpt = (s.vd + 63) / 64;
#define SA_GO(HPW, VPT) return sa_launch<T, HPW, VPT>(q, k_pages, v_pages, tok_seq, tok_pos, table, \
        temperature, bias, lookup, talk, r1, r2, out, n_tokens, s, stream)
    if (hpw <= 1) {
        if (vpt <= 2) SA_GO(1, 2);
        if (vpt <= 8) SA_GO(1, 8);
    } else if (hpw <= 4) {
        if (vpt <= 2) SA_GO(4, 2);
        if (vpt <= 8) SA_GO(4, 8);
    } else if (hpw <= 16) {
        if (vpt <= 2) SA_GO(16, 2);
        if (vpt <= 8) SA_GO(16, 8);
    }
#undef SA_GO
    return (int)hipErrorInvalidValue;
}

extern "C" int gfa_scored_attention(const void* q, const void* k_pages, const void* v_pages,
                                    const int* tok_seq, const int* tok_pos, const int* table,
                                    int table_stride, const float* temperature, const float* bias,
                                    const int* lookup, const float* talk, const float* r1,
                                    const float* r2, int sink, void* out, int n_tokens,
                                    int H, int G, int hd, int vd, long long q_tok, long long q_head,
                                    long long o_tok, long long o_head, float scale, float softcap,
                                    int bias_rows, int n_lookup, int window, int is_bf16,
                                    hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (G <= 0 || H % G || hd <= 0 || vd <= 0 || vd > 512) return (int)hipErrorInvalidValue;
    if ((r1 == nullptr) != (r2 == nullptr)) return (int)hipErrorInvalidValue;
    SAShape s{H, G, hd, vd, q_tok, q_head, o_tok, o_head, table_stride, window, scale, softcap,
              bias_rows, n_lookup, sink ? 1 : 0};
    if (is_bf16)
        return sa_dispatch<bf16_t>(q, k_pages, v_pages, tok_seq, tok_pos, table, temperature, bias,
                                   lookup, talk, r1, r2, out, n_tokens, s, stream);
    return sa_dispatch<float>(q, k_pages, v_pages, tok_seq, tok_pos, table, temperature, bias,
                              lookup, talk, r1, r2, out, n_tokens, s, stream);
}

// --------------------------------------------------------------------------------------
// The same attention for bfloat16 on the matrix cores (head sizes in eights up to 576, value
// sizes in sixteens up to 512).  A wave owns a tile of 16 rows, each a (token, head) pair of
// one kv head, and walks the key blocks of 32 that its rows see.  Both products are formed
// transposed, so that every operand is read in the order the cache has:
//   S^T = K Q^T   A = 16 keys x 32 dims of a key page, B = Q^T from registers;
//   O^T = V^T P^T A = 16 dims x 32 keys of a value page, B = the eight weights a lane holds.
// v_mfma_f32_16x16x32_bf16: lane l supplies row (A) / column (B) l % 16, k = 8 (l / 16) .. +7,
// and receives rows 4 (l / 16) .. +3 of column l % 16; with the key order of common.h those
// rows of the two 16-key tiles are the lane's keys 8 (l / 16) .. +7 of the block.  Scores, the
// steps on them, the softmax and both products' sums are float; the weights are rounded to
// bfloat16 as the second product's operand.
//
// Without a mix across heads the waves of a workgroup are tiles of their own (grid: tiles / 4,
// kv heads, sequences).  With one, the waves of a workgroup are the kv heads of one group of
// tokens (a kv head with more than 16 heads takes several waves): every wave puts its tile of
// scores into shared memory, and every lane adds up, for its row's head and its eight keys,
// the scores of all heads of the same token.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 sa_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float sa_floatx4_t;
union SAFrag {
    uint4 u;
    bf16_t e[8];
    sa_bf16x8_t v;
};

#define SA_SROW 36            // floats per row of a wave's score tile in shared memory (32 + 4)
#define SA_LUT_MAX 8192       // distances whose rows a workgroup with a mix keeps in shared memory

// floats of shared memory before the score tiles of a workgroup with a mix: talk [H][H], the
// distance table [rows][H] and, if it is short enough, the distances' rows
__host__ __device__ inline int sam_tables(int H, int bias_rows, int n_lookup, bool with_bias) {
    int n = (H * H + 3) / 4 * 4;
    if (with_bias) {
        n += (bias_rows * H + 3) / 4 * 4;
        if (n_lookup <= SA_LUT_MAX) n += (n_lookup + 3) / 4 * 4;
    }
    return n;
}

__device__ __forceinline__ float sa_max_lane_groups(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, GFA_WAVE));
    return fmaxf(v, __shfl_xor(v, 32, GFA_WAVE));
}
__device__ __forceinline__ float sa_sum_lane_groups(float v) {
    v += __shfl_xor(v, 16, GFA_WAVE);
    return v + __shfl_xor(v, 32, GFA_WAVE);
}

template <int DK, int DVT, int MAXT, bool SPLIT>
__global__ __launch_bounds__(MAXT) void scored_attention_mfma_kernel(
        const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
        const bf16_t* __restrict__ v_pages, const int* __restrict__ q_start,
        const int* __restrict__ start_pos, const int* __restrict__ table,
        const float* __restrict__ temperature, const float* __restrict__ bias,
        const int* __restrict__ lookup, const float* __restrict__ talk,
        const float* __restrict__ r1, const float* __restrict__ r2, bf16_t* __restrict__ out,
        SAShape s) {
    extern __shared__ __attribute__((aligned(16))) float sam_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int seq = blockIdx.z;
    const int gs = s.H / s.G;
    const int q0 = q_start[seq], q_len = q_start[seq + 1] - q0;
    const int spos = start_pos[seq];
    const int* pages = table + (size_t)seq * s.table_stride;
    const bool mix = talk != nullptr;

    // which (token, head) this lane's row is, and which tokens the wave's rows span
    int g, tok, head, tok_lo, tok_hi;
    bool row_ok;
    if (!mix) {
        g = blockIdx.y;
        const int rows_total = q_len * gs, row0 = (SPLIT ? blockIdx.x : blockIdx.x * nw + wave) * 16;
        if (row0 >= rows_total) return;                // SPLIT: the whole workgroup; else no barrier follows
        row_ok = row0 + li < rows_total;
        const int row = row_ok ? row0 + li : rows_total - 1;
        tok = row / gs;
        head = g * gs + row % gs;
        tok_lo = row0 / gs;
        tok_hi = (row0 + 15 < rows_total ? row0 + 15 : rows_total - 1) / gs;
    } else {
        const int tpg = gs > 16 ? (gs + 15) / 16 : 1, tp = gs > 16 ? 1 : 16 / gs;
        g = wave / tpg;
        tok_lo = blockIdx.x * tp;
        if (tok_lo >= q_len) return;                   // the whole workgroup
        tok_hi = tok_lo + tp - 1 < q_len ? tok_lo + tp - 1 : q_len - 1;
        int hg;
        if (gs > 16) {
            tok = tok_lo;
            hg = (wave % tpg) * 16 + li;
            row_ok = hg < gs;
        } else {
            tok = tok_lo + li / gs;
            hg = li % gs;
            row_ok = li < tp * gs && tok <= tok_hi;
        }
        if (!row_ok) {
            tok = tok_lo;
            hg = 0;
        }
        head = g * gs + hg;
    }
    const int pos = spos + tok;
    const int lo = (s.window > 0 && pos - s.window + 1 > 0) ? pos - s.window + 1 : 0;
    const int pos_max = spos + tok_hi;
    const int lo_min = (s.window > 0 && spos + tok_lo - s.window + 1 > 0) ? spos + tok_lo - s.window + 1 : 0;
    const int last_key = spos + q_len - 1;             // the newest key the cache holds of this sequence

    // with a mix the small tables live in shared memory (the workgroup walks many key blocks
    // and reads them at every one)
    float* talk_lds = sam_lds;                         // [H][H]
    float* tiles = sam_lds + (mix ? sam_tables(s.H, s.bias_rows, s.n_lookup, bias != nullptr) : 0);
    const float* bias_t = bias;                        // [rows][H]
    const int* lookup_t = lookup;
    if (mix) {
        for (int e = threadIdx.x; e < s.H * s.H; e += blockDim.x) talk_lds[e] = talk[e];
        if (bias) {
            float* b_lds = sam_lds + (s.H * s.H + 3) / 4 * 4;
            for (int e = threadIdx.x; e < s.bias_rows * s.H; e += blockDim.x) b_lds[e] = bias[e];
            bias_t = b_lds;
            if (s.n_lookup <= SA_LUT_MAX) {
                int* l_lds = (int*)(b_lds + (s.bias_rows * s.H + 3) / 4 * 4);
                for (int e = threadIdx.x; e < s.n_lookup; e += blockDim.x) l_lds[e] = lookup[e];
                lookup_t = l_lds;
            }
        }
        __syncthreads();
    }

    SAFrag qf[DK];
    const bf16_t* qrow = q + (size_t)(q0 + tok) * s.q_tok + (size_t)head * s.q_head;
#pragma unroll
    for (int kk = 0; kk < DK; ++kk) {
        const int d = kk * 32 + lg * 8;
        qf[kk].u = d < s.hd ? *(const uint4*)(qrow + d) : make_uint4(0, 0, 0, 0);
    }
    const float row_scale = s.scale * (temperature ? temperature[head] : 1.f);
    const float cap_exp = s.softcap > 0.f ? 2.885390081777927f / s.softcap : 0.f;     // 2 log2(e) / cap
    const int vtiles = s.vd / 16;
    sa_floatx4_t o[DVT];
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt) o[dt] = sa_floatx4_t{0.f, 0.f, 0.f, 0.f};
    // a sink is one more key of score zero without a value: the maximum starts at 0 and the
    // sum at 1 (once per row: in one lane group, and in the first wave of a tile's waves)
    const bool sink_here = s.sink && (!SPLIT || wave == 0);
    float m = sink_here ? 0.f : -INFINITY, l = (sink_here && lg == 0) ? 1.f : 0.f;
    const float r1h = r1 ? r1[head] : 0.f, r2h = r1 ? r2[head] : 0.f;

    // SPLIT: the waves of a workgroup share one tile of rows and take its key blocks in turn
    for (int bi = lo_min / 32 + (SPLIT ? wave : 0); bi <= pos_max / 32; bi += SPLIT ? nw : 1) {
        const int page = pages[bi >> 1];
        const bf16_t* kb = k_pages + cache_region(page, g, s.G, s.hd) + (size_t)(bi & 1) * 32 * s.hd;
        const bf16_t* vb = v_pages + cache_region(page, g, s.G, s.vd) + (size_t)(bi & 1) * 512;
        // few value tiles: their loads are asked for with the keys', ahead of the scores' work
        SAFrag vpre[DVT <= 8 ? DVT : 1];
        if (DVT <= 8) {
#pragma unroll
            for (int dt = 0; dt < (DVT <= 8 ? DVT : 1); ++dt) {
                const int dtc = dt < vtiles ? dt : vtiles - 1;
                vpre[dt].u = *(const uint4*)(vb + (size_t)dtc * 1024 + lg * 128 + li * 8);
            }
        }
        sa_floatx4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < DK; ++kk) {
            const int chunk = kk * 4 + lg;
            const int c = chunk * 8 < s.hd ? chunk : 0;          // q is zero there
            const bf16_t* src = kb + c * 256 + li * 8;
            SAFrag k0, k1;
            k0.u = *(const uint4*)src;
            k1.u = *(const uint4*)(src + 128);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0.v, qf[kk].v, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1.v, qf[kk].v, s1, 0, 0, 0);
        }
        float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
        const int key0 = bi * 32 + lg * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int j = key0 + e;
            float v = sv[e] * row_scale;
            // cap tanh(v / cap) = cap (1 - 2 / (e^(2 v / cap) + 1)): one exponential and one
            // reciprocal; exact at both ends, within a few 1e-7 of cap elsewhere
            if (s.softcap > 0.f) v = s.softcap - 2.f * s.softcap * __frcp_rn(exp2f(v * cap_exp) + 1.f);
            if (bias && j <= pos) {
                const int dist = pos - j;
                const int row = dist < s.n_lookup ? lookup_t[dist] : s.bias_rows - 1;
                v += bias_t[(size_t)row * s.H + head];
            }
            if (r1 && j <= pos) v -= r1h * __logf(fmaf(r2h, (float)(pos - j), 1.f));
            // what lies beyond the newest key may be anything: it must not reach the mix
            sv[e] = j <= last_key ? v : 0.f;
        }
        if (mix) {
            float* mine = tiles + ((size_t)wave * 16 + li) * SA_SROW + lg * 8;
            *(float4*)mine = make_float4(sv[0], sv[1], sv[2], sv[3]);
            *(float4*)(mine + 4) = make_float4(sv[4], sv[5], sv[6], sv[7]);
            __syncthreads();
            float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const float* trow = talk_lds + head * s.H;
            // first row of this lane's token in a tile
            const int tok_row = (gs > 16 || !row_ok) ? 0 : (li / gs) * gs;
            // head h2 = g2 gs + r2 of this lane's token is row g2 tpg 16 + tok_row + r2 of the tiles
            const int tpg = gs > 16 ? (gs + 15) / 16 : 1;
            const float* tile_row = tiles + (size_t)tok_row * SA_SROW + lg * 8;
            for (int g2 = 0; g2 < s.G; ++g2) {
                const float* src = tile_row + (size_t)g2 * tpg * 16 * SA_SROW;
                const float* tg = trow + g2 * gs;
#pragma unroll 4
                for (int r2 = 0; r2 < gs; ++r2) {
                    const float4 a = *(const float4*)src, b = *(const float4*)(src + 4);
                    const float t = tg[r2];
                    z[0] = fmaf(t, a.x, z[0]); z[1] = fmaf(t, a.y, z[1]);
                    z[2] = fmaf(t, a.z, z[2]); z[3] = fmaf(t, a.w, z[3]);
                    z[4] = fmaf(t, b.x, z[4]); z[5] = fmaf(t, b.y, z[5]);
                    z[6] = fmaf(t, b.z, z[6]); z[7] = fmaf(t, b.w, z[7]);
                    src += SA_SROW;
                }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) sv[e] = z[e];
            __syncthreads();                           // the tiles are free for the next block
        }
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int j = key0 + e;
            sv[e] = (j <= pos && j >= lo) ? sv[e] * 1.4426950408889634f : -INFINITY;
            mx = fmaxf(mx, sv[e]);
        }
        mx = sa_max_lane_groups(mx);
        const float m_new = fmaxf(m, mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = exp2f(m - m_use);
        SAFrag pf;
        float ps = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = exp2f(sv[e] - m_use);
            ps += p;
            pf.e[e] = float_to_bf16(p);
        }
        l = l * alpha + ps;
        m = m_new;
        // values beyond the newest key: zero bits (their weight is zero, but the pool is not cleared)
        auto two = [&](int e) {
            return (key0 + e <= last_key ? 0xffffu : 0u) | (key0 + e + 1 <= last_key ? 0xffff0000u : 0u);
        };
        const uint4 keep = make_uint4(two(0), two(2), two(4), two(6));
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt) {
            const int dtc = dt < vtiles ? dt : vtiles - 1;
            SAFrag vf;
            if (DVT <= 8) vf.u = vpre[DVT <= 8 ? dt : 0].u;
            else vf.u = *(const uint4*)(vb + (size_t)dtc * 1024 + lg * 128 + li * 8);
            vf.u.x &= keep.x;
            vf.u.y &= keep.y;
            vf.u.z &= keep.z;
            vf.u.w &= keep.w;
            o[dt] *= alpha;
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, o[dt], 0, 0, 0);
        }
    }
    l = sa_sum_lane_groups(l);
    if (SPLIT) {
        // per wave: m and l of its 16 rows, then O^T [dim][row]; the first wave adds them up in
        // wave order (the maxima are in units of log 2)
        const int per_wave = 32 + s.vd * 16;
        float* mine = sam_lds + (size_t)wave * per_wave;
        if (lg == 0) {
            mine[li] = m;
            mine[16 + li] = l;
        }
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt)
            if (dt < vtiles)
#pragma unroll
                for (int j = 0; j < 4; ++j) mine[32 + (dt * 16 + lg * 4 + j) * 16 + li] = o[dt][j];
        __syncthreads();
        if (wave != 0) return;
        float M = -INFINITY;
        for (int w = 0; w < nw; ++w) M = fmaxf(M, sam_lds[(size_t)w * per_wave + li]);
        l = 0.f;
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt) o[dt] = sa_floatx4_t{0.f, 0.f, 0.f, 0.f};
        for (int w = 0; w < nw; ++w) {
            const float* theirs = sam_lds + (size_t)w * per_wave;
            const float mw = theirs[li];
            const float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
            l = fmaf(theirs[16 + li], f, l);
#pragma unroll
            for (int dt = 0; dt < DVT; ++dt)
                if (dt < vtiles)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        o[dt][j] = fmaf(theirs[32 + (dt * 16 + lg * 4 + j) * 16 + li], f, o[dt][j]);
        }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (!row_ok) return;
    bf16_t* orow = out + (size_t)(q0 + tok) * s.o_tok + (size_t)head * s.o_head;
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt) {
        if (dt < vtiles) {
            const uint32_t a = (uint32_t)float_to_bf16(o[dt][0] * inv) | ((uint32_t)float_to_bf16(o[dt][1] * inv) << 16);
            const uint32_t b = (uint32_t)float_to_bf16(o[dt][2] * inv) | ((uint32_t)float_to_bf16(o[dt][3] * inv) << 16);
            uint32_t* dst = (uint32_t*)(orow + dt * 16 + lg * 4);
            dst[0] = a;
            dst[1] = b;
        }
    }
}

template <int DK, int DVT, int MAXT, bool SPLIT>
static int sam_launch(const void* q, const void* k_pages, const void* v_pages, const int* q_start,
                      const int* start_pos, const int* table, const float* temperature,
                      const float* bias, const int* lookup, const float* talk, const float* r1,
                      const float* r2, void* out, int n_seqs, int max_q_len, const SAShape& s,
                      hipStream_t stream) {
    const int gs = s.H / s.G;
    dim3 grid, block;
    size_t shmem = 0;
    if (talk) {
        const int tpg = gs > 16 ? (gs + 15) / 16 : 1, tp = gs > 16 ? 1 : 16 / gs;
        const int waves = s.G * tpg;
        if (waves * 64 > MAXT) return (int)hipErrorInvalidValue;
        grid = dim3((max_q_len + tp - 1) / tp, 1, n_seqs);
        block = dim3(waves * 64);
        shmem = sizeof(float) * ((size_t)sam_tables(s.H, s.bias_rows, s.n_lookup, bias != nullptr)
                                 + (size_t)waves * 16 * SA_SROW);
        if (shmem > 64 * 1024) {
            static bool allowed = false;
            if (!allowed) {
                const hipError_t e = hipFuncSetAttribute(
                    (const void*)scored_attention_mfma_kernel<DK, DVT, MAXT, SPLIT>,
                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return (int)e;
                allowed = true;
            }
        }
    } else if (SPLIT) {
        // as many waves as their partial results fit the shared memory a workgroup may have
        int waves = s.vd > 256 ? 4 : 8;
        if (waves * 64 > MAXT) waves = MAXT / 64;      // the kernel built for fewer, with more registers
        grid = dim3((max_q_len * gs + 15) / 16, s.G, n_seqs);
        block = dim3(waves * 64);
        shmem = sizeof(float) * (size_t)waves * (32 + (size_t)s.vd * 16);
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute(
                (const void*)scored_attention_mfma_kernel<DK, DVT, MAXT, SPLIT>,
                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
    } else {
        const int tiles = (max_q_len * gs + 15) / 16;
        grid = dim3((tiles + 3) / 4, s.G, n_seqs);
        block = dim3(256);
    }
    scored_attention_mfma_kernel<DK, DVT, MAXT, SPLIT><<<grid, block, shmem, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, q_start, start_pos, table,
        temperature, bias, lookup, talk, r1, r2, (bf16_t*)out, s);
    return GFA_LAUNCH_RESULT();
}

// 1 if the matrix-core kernel takes these sizes (bfloat16 only)
extern "C" int gfa_scored_attention_mfma_takes(int H, int G, int hd, int vd, int mixed) {
    if (G <= 0 || H % G || hd % 8 || vd % 16 || hd > 576 || vd > 512 || hd < 8) return 0;
    if (mixed) {
        const int gs = H / G;
        const int waves = G * (gs > 16 ? (gs + 15) / 16 : 1);
        if (H > 64 || (gs <= 16 && 16 / gs < 1)) return 0;
        const bool small = hd <= 128 && vd <= 128;
        if (waves > (small ? 16 : 4)) return 0;
        // talk, a distance table of up to 64 rows and its distances' rows, the tiles
        if (sizeof(float) * ((size_t)H * H + 64 * H + SA_LUT_MAX + 16 + (size_t)waves * 16 * SA_SROW)
                > 150 * 1024) return 0;
    }
    return 1;
}

extern "C" int gfa_scored_attention_mfma(const void* q, const void* k_pages, const void* v_pages,
                                         const int* q_start, const int* start_pos, const int* table,
                                         int table_stride, const float* temperature,
                                         const float* bias, const int* lookup, const float* talk,
                                         const float* r1, const float* r2, int sink,
                                         void* out, int n_seqs, int max_q_len, int H, int G, int hd,
                                         int vd, long long q_tok, long long q_head, long long o_tok,
                                         long long o_head, float scale, float softcap, int bias_rows,
                                         int n_lookup, int window, hipStream_t stream) {
    if (n_seqs <= 0 || max_q_len <= 0) return 0;
    if (!gfa_scored_attention_mfma_takes(H, G, hd, vd, talk != nullptr) || n_seqs > 65535)
        return (int)hipErrorInvalidValue;
    // 16-byte loads of q, 4-byte stores of the result
    if (q_tok % 8 || q_head % 8 || o_tok % 2 || o_head % 2) return (int)hipErrorInvalidValue;
    if ((r1 == nullptr) != (r2 == nullptr)) return (int)hipErrorInvalidValue;
    SAShape s{H, G, hd, vd, q_tok, q_head, o_tok, o_head, table_stride, window, scale, softcap,
              bias_rows, n_lookup, sink ? 1 : 0};
#define SAM_GO(DK, DVT, MAXT, SPLIT) return sam_launch<DK, DVT, MAXT, SPLIT>(q, k_pages, v_pages, q_start, \
        start_pos, table, temperature, bias, lookup, talk, r1, r2, out, n_seqs, max_q_len, s, stream)
    // one token per sequence and no mix: the waves of a workgroup share a tile's key blocks
    if (max_q_len == 1 && talk == nullptr) {
        if (hd <= 128 && vd <= 128) SAM_GO(4, 8, 512, true);
        if (hd <= 256 && vd <= 256) SAM_GO(8, 16, 512, true);
        SAM_GO(18, 32, 256, true);               // four waves: a wave per SIMD has its 512 registers
    }
    if (hd <= 128 && vd <= 128) {
        // the workgroup's size bounds a wave's registers: no larger than the waves of a mix need
        const int gs = H / G;
        const int waves = talk ? G * (gs > 16 ? (gs + 15) / 16 : 1) : 4;
        // (a prompt's many workgroups of eight waves run faster two to a compute unit with 128
        // registers a wave and a few of them in scratch memory - 660 against 748 us for 2,048
        // tokens of 32 heads - than one to a compute unit with all in registers; single-token
        // steps the other way round)
        if (waves <= 4) SAM_GO(4, 8, 256, false);
        if (waves <= 8 && max_q_len <= 16) SAM_GO(4, 8, 512, false);
        SAM_GO(4, 8, 1024, false);
    }
    if (hd <= 256 && vd <= 256) SAM_GO(8, 16, 256, false);
    SAM_GO(18, 32, 256, false);
#undef SAM_GO
}

// --------------------------------------------------------------------------------------
// q, keys and values of attention with unit-norm heads from the projection's float sums:
// a row of proj is [H heads of q | G heads of k | G heads of v] (d, d, dv wide); the bias
// (same layout, optional) is added first; every head of q and k is divided by its root mean
// square (eps inside the root; eps < 0: not normed) and multiplied by a weight per element of
// a head (wq, wk of d elements, shared by the heads; null: not); then the first `rot` elements
// of every head of q and k are turned by pos * freqs[i], pairs (2i, 2i + 1) (layout 0) or
// (i, i + rot / 2) (layout 1), with cos and sin multiplied by `trig` (rot 0: no rotation).
// q goes to q_out [N, H, d]; keys and values to the token's place in the cache (skipped if
// k_pages is null).  One workgroup per token, one wave per head vector, float arithmetic, one
// rounding at the store.
template <typename T>
__global__ __launch_bounds__(SA_THREADS) void unit_heads_store_kernel(
        const float* __restrict__ proj, int row_width, const float* __restrict__ bias,
        T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, int H, int G, int d, int dv, float eps,
        const float* __restrict__ wq, const float* __restrict__ wk,
        const float* __restrict__ freqs, int rot, int layout, float trig) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x;
    const float* row = proj + (size_t)n * row_width;
    const int pos = tok_pos[n];
    const int page = k_pages ? table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE] : 0;
    const int slot = pos % GFA_PAGE;
    const int half = rot >> 1;
    for (int u = wave; u < H + 2 * G; u += SA_WAVES) {
        const bool is_q = u < H, is_k = !is_q && u < H + G;
        const int width = (is_q || is_k) ? d : dv;
        const int off = is_q ? u * d : (is_k ? H * d + (u - H) * d : (H + G) * d + (u - H - G) * dv);
        if (!is_q && !k_pages) continue;
        float r = 1.f;
        if ((is_q || is_k) && eps >= 0.f) {
            float ss = 0.f;
            for (int e = lane; e < width; e += 64) {
                const float x = row[off + e] + (bias ? bias[off + e] : 0.f);
                ss = fmaf(x, x, ss);
            }
            r = rsqrtf(wave_sum(ss) / (float)width + eps);
        }
        const float* hw = is_q ? wq : (is_k ? wk : nullptr);
        for (int e = lane; e < width; e += 64) {
            float x = (row[off + e] + (bias ? bias[off + e] : 0.f)) * r * (hw ? hw[e] : 1.f);
            if ((is_q || is_k) && e < rot) {
                // the element's partner in its pair, normed the same way
                const bool first = layout == 0 ? (e & 1) == 0 : e < half;
                const int p = layout == 0 ? (e ^ 1) : (first ? e + half : e - half);
                const float y = (row[off + p] + (bias ? bias[off + p] : 0.f)) * r * (hw ? hw[p] : 1.f);
                float sn, cs;
                sincosf((float)pos * freqs[layout == 0 ? e >> 1 : (first ? e : e - half)], &sn, &cs);
                x = first ? (x * cs - y * sn) * trig : (x * cs + y * sn) * trig;
            }
            if (is_q) store_from_float(q_out + ((size_t)n * H + u) * d + e, x);
            else if (is_k) store_from_float(k_pages + key_elem(page, u - H, slot, e, G, d), x);
            else store_from_float(v_pages + value_elem(page, u - H - G, e, slot, G, dv), x);
        }
    }
}

extern "C" int gfa_unit_heads_store(const float* proj, int row_width, const float* bias, void* q_out,
                                    void* k_pages, void* v_pages, const int* tok_seq,
                                    const int* tok_pos, const int* table, int table_stride,
                                    int n_tokens, int H, int G, int d, int dv, float eps,
                                    const float* wq, const float* wk, const float* freqs, int rot,
                                    int layout, float trig, int is_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rot < 0 || rot > d || rot % 2 || (rot && !freqs) || (layout != 0 && layout != 1))
        return (int)hipErrorInvalidValue;
    if (is_bf16)
        unit_heads_store_kernel<bf16_t><<<n_tokens, SA_THREADS, 0, stream>>>(
            proj, row_width, bias, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, tok_seq,
            tok_pos, table, table_stride, H, G, d, dv, eps, wq, wk, freqs, rot, layout, trig);
    else
        unit_heads_store_kernel<float><<<n_tokens, SA_THREADS, 0, stream>>>(
            proj, row_width, bias, (float*)q_out, (float*)k_pages, (float*)v_pages, tok_seq,
            tok_pos, table, table_stride, H, G, d, dv, eps, wq, wk, freqs, rot, layout, trig);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// q, keys and values of attention whose q and k are normed over the WHOLE projection, from the
// projection's float sums: a row of proj is [H heads of q | G heads of k | G heads of v]
// (d, d, dv wide; with values_are_keys there is no v part and a kv head's value is its key as
// projected, bias added, before the norm, so dv = d).  The bias (layout of the row, optional)
// is added first; all of q is divided by its root mean square over H d elements and
// multiplied by wq, all of k likewise over G d elements with wk (eps inside the root; eps < 0:
// not normed, no weights); q is then multiplied by 1 + temp_coef ln(floor((pos + 1) /
// temp_every) + 1) (temp_every 0: not).  q goes to q_out [N, H, d]; keys and values to the
// token's place in the cache (skipped if k_pages is null).  One workgroup per token, float
// arithmetic, one rounding at the store.
template <typename T>
__global__ __launch_bounds__(SA_THREADS) void whole_norm_store_kernel(
        const float* __restrict__ proj, int row_width, const float* __restrict__ bias,
        const float* __restrict__ wq, const float* __restrict__ wk, T* __restrict__ q_out,
        T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ tok_seq,
        const int* __restrict__ tok_pos, const int* __restrict__ table, int table_stride, int H,
        int G, int d, int dv, float eps, float temp_coef, int temp_every, int values_are_keys) {
    __shared__ float scratch[16];
    const int n = blockIdx.x;
    const float* row = proj + (size_t)n * row_width;
    const int pos = tok_pos[n];
    const int nq = H * d, nk = G * d;
    float rq = 1.f, rk = 1.f;
    if (eps >= 0.f) {
        float ss = 0.f;
        for (int e = threadIdx.x; e < nq; e += SA_THREADS) {
            const float x = row[e] + (bias ? bias[e] : 0.f);
            ss = fmaf(x, x, ss);
        }
        rq = rsqrtf(block_sum(ss, scratch) / (float)nq + eps);
        ss = 0.f;
        for (int e = threadIdx.x; e < nk; e += SA_THREADS) {
            const float x = row[nq + e] + (bias ? bias[nq + e] : 0.f);
            ss = fmaf(x, x, ss);
        }
        rk = rsqrtf(block_sum(ss, scratch) / (float)nk + eps);
    }
    if (temp_every > 0) rq *= 1.f + temp_coef * logf((float)((pos + 1) / temp_every + 1));
    for (int e = threadIdx.x; e < nq; e += SA_THREADS) {
        const float x = row[e] + (bias ? bias[e] : 0.f);
        store_from_float(q_out + (size_t)n * nq + e, x * rq * (eps >= 0.f ? wq[e] : 1.f));
    }
    if (!k_pages) return;
    const int page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int slot = pos % GFA_PAGE;
    for (int e = threadIdx.x; e < nk; e += SA_THREADS) {
        const float x = row[nq + e] + (bias ? bias[nq + e] : 0.f);
        const int g = e / d, i = e - g * d;
        store_from_float(k_pages + key_elem(page, g, slot, i, G, d), x * rk * (eps >= 0.f ? wk[e] : 1.f));
        if (values_are_keys) store_from_float(v_pages + value_elem(page, g, i, slot, G, dv), x);
    }
    if (!values_are_keys) {
        for (int e = threadIdx.x; e < G * dv; e += SA_THREADS) {
            const float x = row[nq + nk + e] + (bias ? bias[nq + nk + e] : 0.f);
            const int g = e / dv, i = e - g * dv;
            store_from_float(v_pages + value_elem(page, g, i, slot, G, dv), x);
        }
    }
}

extern "C" int gfa_whole_norm_store(const float* proj, int row_width, const float* bias,
                                    const float* wq, const float* wk, void* q_out, void* k_pages,
                                    void* v_pages, const int* tok_seq, const int* tok_pos,
                                    const int* table, int table_stride, int n_tokens, int H, int G,
                                    int d, int dv, float eps, float temp_coef, int temp_every,
                                    int values_are_keys, int is_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if ((values_are_keys && dv != d) || (eps >= 0.f && (!wq || !wk)) || temp_every < 0)
        return (int)hipErrorInvalidValue;
    if (is_bf16)
        whole_norm_store_kernel<bf16_t><<<n_tokens, SA_THREADS, 0, stream>>>(
            proj, row_width, bias, wq, wk, (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages,
            tok_seq, tok_pos, table, table_stride, H, G, d, dv, eps, temp_coef, temp_every,
            values_are_keys);
    else
        whole_norm_store_kernel<float><<<n_tokens, SA_THREADS, 0, stream>>>(
            proj, row_width, bias, wq, wk, (float*)q_out, (float*)k_pages, (float*)v_pages,
            tok_seq, tok_pos, table, table_stride, H, G, d, dv, eps, temp_coef, temp_every,
            values_are_keys);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The latents of latent attention from the float sums of the token's two down projections:
// a row of proj is [q latent (q_rank) | kv latent (R) | key part to rotate (dr)].
//   cq_out[n, :] = rmsnorm(q latent) * wq              (operand of the query's up projection)
//   c = rmsnorm(kv latent) * wkv  -> the cache's key elements 0 .. R-1 and value elements 0 .. R-1
//   rotated part: pairs (2i, 2i+1), i < rotary_dim / 2, turned by pos * freqs[i], the rest as
//   it is -> the cache's key elements R .. R+dr-1
// The cache has one kv head with keys of R + dr and values of R.  One workgroup per token.
template <typename T>
__global__ __launch_bounds__(SA_THREADS) void latent_store_kernel(
        const float* __restrict__ proj, int row_width, int q_rank, int R, int dr,
        const float* __restrict__ wq, const float* __restrict__ wkv, float eps,
        const float* __restrict__ freqs, int rotary_dim, T* __restrict__ cq_out,
        T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ tok_seq,
        const int* __restrict__ tok_pos, const int* __restrict__ table, int table_stride) {
    __shared__ float scratch[16];
    const int n = blockIdx.x;
    const float* row = proj + (size_t)n * row_width;
    const int pos = tok_pos[n];
    float ss = 0.f;
    if (q_rank > 0) {                                  // q_rank 0: the query has no latent
        for (int e = threadIdx.x; e < q_rank; e += SA_THREADS) ss = fmaf(row[e], row[e], ss);
        const float rq = rsqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
        for (int e = threadIdx.x; e < q_rank; e += SA_THREADS)
            store_from_float(cq_out + (size_t)n * q_rank + e, row[e] * rq * wq[e]);
    }
    if (!k_pages) return;
    const float* kv = row + q_rank;
    ss = 0.f;
    for (int e = threadIdx.x; e < R; e += SA_THREADS) ss = fmaf(kv[e], kv[e], ss);
    const float rc = rsqrtf(block_sum(ss, scratch) / (float)R + eps);
    const int page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int slot = pos % GFA_PAGE;
    const int hd = R + dr;
    for (int e = threadIdx.x; e < R; e += SA_THREADS) {
        const float c = kv[e] * rc * wkv[e];
        store_from_float(k_pages + key_elem(page, 0, slot, e, 1, hd), c);
        store_from_float(v_pages + value_elem(page, 0, e, slot, 1, R), c);
    }
    const float* kr = kv + R;
    for (int i = threadIdx.x; i < dr / 2; i += SA_THREADS) {
        float u = kr[2 * i], v = kr[2 * i + 1];
        if (2 * i < rotary_dim) {
            float sn, cs;
            sincosf((float)pos * freqs[i], &sn, &cs);
            const float u2 = u * cs - v * sn, v2 = v * cs + u * sn;
            u = u2;
            v = v2;
        }
        store_from_float(k_pages + key_elem(page, 0, slot, R + 2 * i, 1, hd), u);
        store_from_float(k_pages + key_elem(page, 0, slot, R + 2 * i + 1, 1, hd), v);
    }
    if ((dr & 1) && threadIdx.x == 0)
        store_from_float(k_pages + key_elem(page, 0, slot, hd - 1, 1, hd), kr[dr - 1]);
}

extern "C" int gfa_latent_store(const float* proj, int row_width, int q_rank, int R, int dr,
                                const float* wq, const float* wkv, float eps, const float* freqs,
                                int rotary_dim, void* cq_out, void* k_pages, void* v_pages,
                                const int* tok_seq, const int* tok_pos, const int* table,
                                int table_stride, int n_tokens, int is_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rotary_dim % 2 || rotary_dim > dr) return (int)hipErrorInvalidValue;
    if (is_bf16)
        latent_store_kernel<bf16_t><<<n_tokens, SA_THREADS, 0, stream>>>(
            proj, row_width, q_rank, R, dr, wq, wkv, eps, freqs, rotary_dim, (bf16_t*)cq_out,
            (bf16_t*)k_pages, (bf16_t*)v_pages, tok_seq, tok_pos, table, table_stride);
    else
        latent_store_kernel<float><<<n_tokens, SA_THREADS, 0, stream>>>(
            proj, row_width, q_rank, R, dr, wq, wkv, eps, freqs, rotary_dim, (float*)cq_out,
            (float*)k_pages, (float*)v_pages, tok_seq, tok_pos, table, table_stride);
    return GFA_LAUNCH_RESULT();
}

// The query of latent attention from the float sums of its up projection, a row of
// [H heads of (d plain | dr to rotate)]: the plain parts go head by head to
// plain_out [H, N, d] (operand of the product with the keys' up projection), the rotated
// parts to elements R .. R+dr-1 of full_out [H, N, R + dr], whose first R elements that
// product fills.  A token's row starts q_stride floats after the one before.  grid (tokens, heads).
template <typename T>
__global__ void latent_query_kernel(const float* __restrict__ q, const float* __restrict__ freqs,
                                    int rotary_dim, const int* __restrict__ tok_pos,
                                    T* __restrict__ plain_out, T* __restrict__ full_out, int N, int H,
                                    int d, int dr, int R, long long q_stride) {
    const int n = blockIdx.x, h = blockIdx.y;
    const float* row = q + (size_t)n * q_stride + (size_t)h * (d + dr);
    T* plain = plain_out + ((size_t)h * N + n) * d;
    for (int e = threadIdx.x; e < d; e += blockDim.x) store_from_float(plain + e, row[e]);
    T* full = full_out + ((size_t)h * N + n) * (R + dr) + R;
    const float* qr = row + d;
    const int pos = tok_pos[n];
    for (int i = threadIdx.x; i < dr / 2; i += blockDim.x) {
        float u = qr[2 * i], v = qr[2 * i + 1];
        if (2 * i < rotary_dim) {
            float sn, cs;
            sincosf((float)pos * freqs[i], &sn, &cs);
            const float u2 = u * cs - v * sn, v2 = v * cs + u * sn;
            u = u2;
            v = v2;
        }
        store_from_float(full + 2 * i, u);
        store_from_float(full + 2 * i + 1, v);
    }
    if ((dr & 1) && threadIdx.x == 0) store_from_float(full + dr - 1, qr[dr - 1]);
}

extern "C" int gfa_latent_query(const float* q, const float* freqs, int rotary_dim,
                                const int* tok_pos, void* plain_out, void* full_out, int n_tokens,
                                int H, int d, int dr, int R, long long q_stride, int is_bf16,
                                hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (H > 65535 || rotary_dim % 2 || rotary_dim > dr || q_stride < (long long)H * (d + dr))
        return (int)hipErrorInvalidValue;
    dim3 grid(n_tokens, H);
    if (is_bf16)
        latent_query_kernel<bf16_t><<<grid, 64, 0, stream>>>(q, freqs, rotary_dim, tok_pos,
                                                             (bf16_t*)plain_out, (bf16_t*)full_out,
                                                             n_tokens, H, d, dr, R, q_stride);
    else
        latent_query_kernel<float><<<grid, 64, 0, stream>>>(q, freqs, rotary_dim, tok_pos,
                                                            (float*)plain_out, (float*)full_out,
                                                            n_tokens, H, d, dr, R, q_stride);
    return GFA_LAUNCH_RESULT();
}
