// Latent attention: every token caches ONE vector c (kv_rank values); a head's keys and values are linear maps of it.
// The maps are folded into the query and the output, so the kernel attends over the cached latents themselves:
//     score_j = scale * q~ . c_j   (q~ = the head's key map transposed, applied to its query),   o~ = sum_j p_j c_j
// and the head's output is its value map applied to o~.  All heads of a token share the same keys, and a key row
// serves as the value row too.  Scores, softmax weights and the weighted sum are float32; the cache holds the
// activations' format (`fmt`: 0 bfloat16, 1 float16, 2 float32).  No positions enter.
#include "nvx_dev.h"

namespace NVX_NS {

template <typename A> __device__ __forceinline__ float la_ld(const A* p, int64_t i) { return (float)p[i]; }
template <typename A> __device__ __forceinline__ void la_st(A* p, int64_t i, float v) { p[i] = (A)v; }

__device__ __forceinline__ float la_block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// ---- what follows the down projections --------------------------------------------------------------------------------
// x[t] = [ query latent (q_rank) | key/value latent (kv_rank) | one output-gate pre-activation per head ].
//   cq[t]           = query latent / rms * w_q                     (activation format, feeds the query up-projection)
//   cache[slot[t]]  = key/value latent / rms * w_kv                (a negative slot: not stored)
//   gate[t][h]      = sigmoid(pre-activation)                      (float32)
template <typename A>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const A* __restrict__ x, int64_t x_stride, const float* __restrict__ w_q, const float* __restrict__ w_kv, float eps,
    const int64_t* __restrict__ slots, A* __restrict__ cq, A* __restrict__ cache, int64_t n_slots, float* __restrict__ gate,
    int q_rank, int kv_rank, int heads) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const A* r = x + t * x_stride;
    float ss = 0.f;
    for (int c = threadIdx.x; c < q_rank; c += 256) { const float v = la_ld(r, c); ss += v * v; }
    const float rq = 1.0f / sqrtf(la_block_sum(ss, red) / (float)q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += 256) la_st(cq, t * q_rank + c, la_ld(r, c) * rq * w_q[c]);
    ss = 0.f;
    for (int c = threadIdx.x; c < kv_rank; c += 256) { const float v = la_ld(r, q_rank + c); ss += v * v; }
    const float rk = 1.0f / sqrtf(la_block_sum(ss, red) / (float)kv_rank + eps);
    const int64_t slot = slots[t];
    if (slot >= 0 && slot < n_slots)
        for (int c = threadIdx.x; c < kv_rank; c += 256) la_st(cache, slot * kv_rank + c, la_ld(r, q_rank + c) * rk * w_kv[c]);
    for (int h = threadIdx.x; h < heads; h += 256)
        gate[t * heads + h] = 1.0f / (1.0f + expf(-la_ld(r, q_rank + kv_rank + h)));
}

// ---- the same place for a latent with a rotated key part ---------------------------------------------------------------------
// x[t] holds, at their offsets: the queries (heads x [dim plain | rot rotated]), the down projection [latent (kv_rank) | one rotated
// key part (rot) that all heads share], one output-gate pre-activation per head.
//   q_out[t]        = the queries, their rotated parts turned by the token's position
//   cache[slot[t]]  = [ latent / rms * w_kv | key part turned by the position | zeros up to row_len ]
//   gate[t][h]      = sigmoid(pre-activation)                      (float32)
// Pairs are neighbours (2i, 2i + 1); the angle position * freq[i] is formed and brought into [-pi, pi] in double precision (freq:
// float64, rot / 2), cosine and sine are float32 and multiplied by `mag`.  The cache row is a key row for the folded queries
// [W_uk^T q_plain | q_rotated] and its latent part the value row, so the attention over latents serves this layout as it is.
template <typename A>
__global__ __launch_bounds__(256) void latent_rope_prep_kernel(
    const A* __restrict__ x, int64_t x_stride, int q_off, int kv_off, int g_off, const int64_t* __restrict__ positions,
    const double* __restrict__ freq, float mag, const float* __restrict__ w_kv, float eps, const int64_t* __restrict__ slots,
    A* __restrict__ q_out, A* __restrict__ cache, int64_t n_slots, int row_len, float* __restrict__ gate, int heads, int dim, int rot,
    int kv_rank) {
    extern __shared__ float cs[];                // rot: cos | sin
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const A* r = x + t * x_stride;
    const int half = rot / 2;
    const double pos = (double)positions[t];
    for (int i = threadIdx.x; i < half; i += 256) {
        const double two_pi = 6.283185307179586476925286766559;
        const double a = pos * freq[i];
        float sn, c;
        sincosf((float)(a - two_pi * rint(a / two_pi)), &sn, &c);
        cs[i] = c * mag;
        cs[half + i] = sn * mag;
    }
    float ss = 0.f;
    for (int c = threadIdx.x; c < kv_rank; c += 256) { const float v = la_ld(r, kv_off + c); ss += v * v; }
    const float rk = 1.0f / sqrtf(la_block_sum(ss, red) / (float)kv_rank + eps);        // (its barriers also publish cs)
    const int hd = dim + rot;
    for (int i = threadIdx.x; i < heads * hd; i += 256) {
        const int d = i % hd - dim;
        float v = la_ld(r, q_off + i);
        if (d >= 0) {
            const int m = d >> 1;
            v = (d & 1) ? v * cs[m] + la_ld(r, q_off + i - 1) * cs[half + m] : v * cs[m] - la_ld(r, q_off + i + 1) * cs[half + m];
        }
        la_st(q_out, t * (int64_t)heads * hd + i, v);
    }
    for (int h = threadIdx.x; h < heads; h += 256) gate[t * heads + h] = 1.0f / (1.0f + expf(-la_ld(r, g_off + h)));
    const int64_t slot = slots[t];
    if (slot < 0 || slot >= n_slots) return;
    A* row = cache + slot * row_len;
    for (int c = threadIdx.x; c < row_len; c += 256) {
        float v = 0.f;
        if (c < kv_rank) v = la_ld(r, kv_off + c) * rk * w_kv[c];
        else if (c < kv_rank + rot) {
            const int d = c - kv_rank, m = d >> 1;
            const float own = la_ld(r, kv_off + c);
            v = (d & 1) ? own * cs[m] + la_ld(r, kv_off + c - 1) * cs[half + m] : own * cs[m] - la_ld(r, kv_off + c + 1) * cs[half + m];
        }
        la_st(row, c, v);
    }
}

// ---- attention over the cached latents ------------------------------------------------------------------------------
// One workgroup per (query token, group of HG heads).  Keys come in tiles of 256: first every thread scores one key
// against the group's folded queries (held in LDS), the tile's weights go to LDS, then every thread owns output
// columns and adds the tile's weighted rows.  Running maximum and sum per head (online softmax).
// q / out: (heads, tokens, rank).  Token t of sequence b sees the sequence's keys 0 .. kv_len[b] - q_len[b] + local(t).
// kv_indices + kv_start[b]: the slots of sequence b's tokens in order (a flat list with offsets, or rows of a table).
#define LA_KT 256
#define LA_MAXC 4      // output columns per thread: rank <= 256 * LA_MAXC

template <typename A, int HG>
__global__ __launch_bounds__(256) void latent_attn_kernel(
    const A* __restrict__ q, const A* __restrict__ cache, const int32_t* __restrict__ kv_indices, const int64_t* __restrict__ kv_start,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ tok_seq,
    const float* __restrict__ gate, A* __restrict__ out, int heads, int rank, int64_t n_tok, float scale) {
    extern __shared__ float lds[];
    float* q_l = lds;                          // HG * rank
    float* p_l = q_l + HG * rank;              // LA_KT * HG
    int* slot_l = (int*)(p_l + LA_KT * HG);    // LA_KT
    float* red = (float*)(slot_l + LA_KT);     // 4 * HG
    const int64_t t = blockIdx.x;
    const int h0 = blockIdx.y * HG;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const int64_t q0 = qo_indptr ? qo_indptr[b] : t;
    const int64_t q_len = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
    const int64_t n_keys = (int64_t)kv_len[b] - q_len + (t - q0) + 1;
    const int32_t* idx = kv_indices + kv_start[b];
    for (int i = tid; i < HG * rank; i += 256) {
        const int h = h0 + i / rank;
        q_l[i] = h < heads ? la_ld(q, ((int64_t)h * n_tok + t) * rank + (i % rank)) : 0.f;
    }
    float m_run[HG], l_run[HG], acc[LA_MAXC][HG];
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        m_run[h] = -INFINITY;
        l_run[h] = 0.f;
#pragma unroll
        for (int k = 0; k < LA_MAXC; ++k) acc[k][h] = 0.f;
    }
    for (int64_t k0 = 0; k0 < n_keys; k0 += LA_KT) {
        const int64_t j = k0 + tid;
        const bool valid = j < n_keys;
        const int slot = valid ? idx[j] : 0;
        __syncthreads();                                   // q_l is written; the previous tile's p_l and slot_l are read
        slot_l[tid] = slot;
        float s[HG];
#pragma unroll
        for (int h = 0; h < HG; ++h) s[h] = 0.f;
        if (valid) {
            const A* row = cache + (int64_t)slot * rank;
            for (int r = 0; r < rank; ++r) {
                const float c = la_ld(row, r);
#pragma unroll
                for (int h = 0; h < HG; ++h) s[h] += q_l[h * rank + r] * c;
            }
        }
        // tile maximum per head
        float alpha[HG];
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            s[h] = valid ? s[h] * scale : -INFINITY;
            const float wm = wave_max(s[h]);
            if (lane == 0) red[wv * HG + h] = wm;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const float tm = fmaxf(fmaxf(red[h], red[HG + h]), fmaxf(red[2 * HG + h], red[3 * HG + h]));
            const float m_new = fmaxf(m_run[h], tm);       // finite: every tile has at least one visible key
            alpha[h] = expf(m_run[h] - m_new);              // first tile: exp(-inf) = 0
            m_run[h] = m_new;
            s[h] = valid ? expf(s[h] - m_new) : 0.f;
            p_l[tid * HG + h] = s[h];
        }
        __syncthreads();                                   // p_l and slot_l are complete; red has been read
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const float ws = wave_sum(s[h]);
            if (lane == 0) red[wv * HG + h] = ws;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            l_run[h] = l_run[h] * alpha[h] + (red[h] + red[HG + h] + red[2 * HG + h] + red[3 * HG + h]);
#pragma unroll
            for (int k = 0; k < LA_MAXC; ++k) acc[k][h] *= alpha[h];
        }
        const int n_here = (int)((n_keys - k0) < LA_KT ? (n_keys - k0) : LA_KT);
        for (int jj = 0; jj < n_here; ++jj) {
            const A* row = cache + (int64_t)slot_l[jj] * rank;
#pragma unroll
            for (int k = 0; k < LA_MAXC; ++k) {
                const int c = tid + k * 256;
                if (c < rank) {
                    const float v = la_ld(row, c);
#pragma unroll
                    for (int h = 0; h < HG; ++h) acc[k][h] += p_l[jj * HG + h] * v;
                }
            }
        }
    }
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        if (h0 + h >= heads) continue;
        const float f = (gate ? gate[t * heads + h0 + h] : 1.0f) / l_run[h];
#pragma unroll
        for (int k = 0; k < LA_MAXC; ++k) {
            const int c = tid + k * 256;
            if (c < rank) la_st(out, ((int64_t)(h0 + h) * n_tok + t) * rank + c, acc[k][h] * f);
        }
    }
}

// ---- the same on the matrix cores (16-bit formats; rank 32 .. 256 in steps of 32, 320, 384, 448 or 512) -----------------------------------
// One workgroup per (query token, group of 16 heads); its four waves take every fourth tile of 16 keys and merge at the
// end.  Per tile:
//   S^T (16 keys x 16 heads) = C_tile (16 x rank) . Q~^T (rank x 16)        v_mfma_f32_16x16x32, rank / 32 of them; the A
//       operand is read straight from the cache rows (lane (key, quarter) takes 16 bytes per k-step) and parked in LDS;
//   the result leaves every lane with one head (lane & 15) and four keys (4 * quarter + r): the running maximum and sum of
//       a head are kept per lane, reduced over the quarters where needed;
//   O^T (rank x 16 heads) += C_tile^T (rank x 16 keys) . P^T (16 keys x 16 heads)   v_mfma_f32_16x16x16, 32 columns a pair:
//       the pair's A operands are the even and the odd columns, so one 4-byte LDS read (key 4 * quarter + r, columns
//       2 i and 2 i + 1 of the 32) feeds both; P^T is exactly what the lane holds.  The weights stay float32 up to here
//       and enter as hi + lo (two products), which keeps 16 bits of their mantissa.
// Scores, maximum, exponentials and sums are float32.
typedef __attribute__((ext_vector_type(4))) short la_s16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 la_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 la_f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 la_f16x4;

template <typename A> __device__ __forceinline__ nvx_f32x4 la_mfma32(nvx_u32x4 a, nvx_u32x4 b, nvx_f32x4 c) {
    if constexpr (sizeof(A) == 2 && __is_same(A, __bf16))
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(la_bf16x8, a), __builtin_bit_cast(la_bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(la_f16x8, a), __builtin_bit_cast(la_f16x8, b), c, 0, 0, 0);
}
template <typename A> __device__ __forceinline__ nvx_f32x4 la_mfma16(uint2 a, uint2 b, nvx_f32x4 c) {
    if constexpr (__is_same(A, __bf16))
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(la_s16x4, a), __builtin_bit_cast(la_s16x4, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(la_f16x4, a), __builtin_bit_cast(la_f16x4, b), c, 0, 0, 0);
}
template <typename A> __device__ __forceinline__ uint32_t la_pack2(float lo, float hi) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    typedef A a2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, a2));
}
template <typename A> __device__ __forceinline__ float la_round(float v) { return (float)(A)v; }

#define LA_PAD 8     // elements between the rows of a parked tile: 16-byte rows, and the four quarters hit different banks

template <typename A, int RKM>      // RKM = rank / 32, the k-steps of a score product (compile time: the loops below unroll into
                                    // straight-line code, so the LDS reads of a tile run ahead of the products that use them)
__global__ __launch_bounds__(256, (RKM <= 8 ? 2 : 1)) void latent_attn_mfma_kernel(     // up to rank 256: two waves a SIMD
    const A* __restrict__ q, const A* __restrict__ cache, const int32_t* __restrict__ kv_indices, const int64_t* __restrict__ kv_start,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ tok_seq,
    const float* __restrict__ gate, A* __restrict__ out, int heads, int rank, int64_t n_tok, float scale, int skip_groups) {
    extern __shared__ float lds[];
    constexpr int NB2 = RKM;                   // pairs of 16-column blocks = rank / 32
    constexpr int steps = RKM;
    const int64_t t = blockIdx.x;
    if (skip_groups) {                         // tokens whose group of four lies in one sequence belong to the tile kernel below
        const int64_t g0 = t & ~(int64_t)3;
        if (g0 + 3 < n_tok && tok_seq[g0] == tok_seq[g0 + 3]) return;
    }
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, l16 = lane & 15, quarter = lane >> 4;
    const int head = blockIdx.y * 16 + l16;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const int64_t q0 = qo_indptr ? qo_indptr[b] : t;
    const int64_t q_len = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
    const int64_t n_keys = (int64_t)kv_len[b] - q_len + (t - q0) + 1;
    const int32_t* idx = kv_indices + kv_start[b];
    const int row_elems = rank + LA_PAD;
    uint16_t* tile = reinterpret_cast<uint16_t*>(lds) + (size_t)wv * 16 * row_elems;     // this wave's parked tile

    nvx_u32x4 qb[RKM];
#pragma unroll
    for (int ks = 0; ks < RKM; ++ks) {
        qb[ks] = nvx_u32x4{0u, 0u, 0u, 0u};
        if (head < heads)
            qb[ks] = *reinterpret_cast<const nvx_u32x4*>(q + ((int64_t)head * n_tok + t) * rank + 32 * ks + 8 * quarter);
    }
    nvx_f32x4 o_acc[2 * NB2];
#pragma unroll
    for (int i = 0; i < 2 * NB2; ++i) o_acc[i] = nvx_f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;      // of head l16; l_run: this quarter's keys only

    const int64_t n_tiles = (n_keys + 15) >> 4;
    // A tile's rows hang on its slot ids, which hang on the table: two memory round trips in a row.  The ids are read two
    // tiles ahead and the rows one tile ahead, so that neither wait stands in front of a tile's products.
    nvx_u32x4 a_nxt[RKM];
    auto slot_of = [&](int64_t j) {
        const int64_t key = j * 16 + l16;
        return idx[key < n_keys ? key : 0];                      // a key past the end reads a real row and is masked below
    };
    auto fetch = [&](int slot) {
        const A* row = cache + (int64_t)slot * rank;
#pragma unroll
        for (int ks = 0; ks < RKM; ++ks)
            a_nxt[ks] = *reinterpret_cast<const nvx_u32x4*>(row + 32 * ks + 8 * quarter);
    };
    int slot_nxt = 0;
    if (wv < n_tiles) fetch(slot_of(wv));
    if (wv + 4 < n_tiles) slot_nxt = slot_of(wv + 4);
    for (int64_t j = wv; j < n_tiles; j += 4) {
        nvx_u32x4 a_cur[RKM];
#pragma unroll
        for (int ks = 0; ks < RKM; ++ks) a_cur[ks] = a_nxt[ks];
        if (j + 4 < n_tiles) fetch(slot_nxt);
        if (j + 8 < n_tiles) slot_nxt = slot_of(j + 8);
        nvx_f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < RKM; ++ks) {
            *reinterpret_cast<nvx_u32x4*>(tile + l16 * row_elems + 32 * ks + 8 * quarter) = a_cur[ks];
            sacc = la_mfma32<A>(a_cur[ks], qb[ks], sacc);
        }
        // the tile is parked before any lane reads it back transposed (one wave: its LDS operations complete in order);
        // the barrier is for the compiler, which must not move the reads below above the writes
        asm volatile("" ::: "memory");
        float sv[4], mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            sv[r] = (j * 16 + 4 * quarter + r) < n_keys ? sacc[r] * scale : -INFINITY;
            mx = fmaxf(mx, sv[r]);
        }
        mx = fmaxf(mx, xor16(mx));
        mx = fmaxf(mx, xor32(mx));
        const float m_new = fmaxf(m_run, mx);                    // finite: a tile has at least one visible key
        const float alpha = __expf(m_run - m_new);
        const bool rescale = __any(alpha != 1.0f);               // once the maxima have settled, most tiles change none
        m_run = m_new;
        l_run *= alpha;
        float p[4], ph[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = __expf(sv[r] - m_new);
            l_run += p[r];
            ph[r] = la_round<A>(p[r]);
        }
        const uint2 p_hi = make_uint2(la_pack2<A>(ph[0], ph[1]), la_pack2<A>(ph[2], ph[3]));
        const uint2 p_lo = make_uint2(la_pack2<A>(p[0] - ph[0], p[1] - ph[1]), la_pack2<A>(p[2] - ph[2], p[3] - ph[3]));
        const uint32_t* tile32 = reinterpret_cast<const uint32_t*>(tile);
#pragma unroll
        for (int b2 = 0; b2 < NB2; ++b2) {
            {
                uint32_t d[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) d[r] = tile32[((4 * quarter + r) * row_elems + 32 * b2) / 2 + l16];
                const uint2 even = make_uint2((d[0] & 0xffffu) | (d[1] << 16), (d[2] & 0xffffu) | (d[3] << 16));
                const uint2 odd = make_uint2((d[0] >> 16) | (d[1] & 0xffff0000u), (d[2] >> 16) | (d[3] & 0xffff0000u));
                if (rescale) {
                    o_acc[2 * b2] *= alpha;
                    o_acc[2 * b2 + 1] *= alpha;
                }
                o_acc[2 * b2] = la_mfma16<A>(even, p_hi, o_acc[2 * b2]);
                o_acc[2 * b2] = la_mfma16<A>(even, p_lo, o_acc[2 * b2]);
                o_acc[2 * b2 + 1] = la_mfma16<A>(odd, p_hi, o_acc[2 * b2 + 1]);
                o_acc[2 * b2 + 1] = la_mfma16<A>(odd, p_lo, o_acc[2 * b2 + 1]);
            }
        }
        asm volatile("" ::: "memory");                          // (compiler) the reads stay above the next tile's writes
    }

    // merge the four waves' partial results: 2 and 3 into 0 and 1, then 1 into 0.  Every lane parks its own values; the lane
    // of the same number in the other wave holds the same head and columns.
    constexpr int vals = 8 * steps + 2;
    auto park = [&](int region) {
        float* base = lds + (size_t)region * vals * 64 + lane;
#pragma unroll
        for (int i = 0; i < 2 * NB2; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) base[(4 * i + r) * 64] = o_acc[i][r];
        }
        base[(8 * steps) * 64] = m_run;
        base[(8 * steps + 1) * 64] = l_run;
    };
    auto take = [&](int region) {
        const float* base = lds + (size_t)region * vals * 64 + lane;
        const float m_o = base[(8 * steps) * 64], l_o = base[(8 * steps + 1) * 64];
        const float m_new = fmaxf(m_run, m_o);
        const float ref = m_new == -INFINITY ? 0.f : m_new;
        const float fa = __expf(m_run - ref), fb = __expf(m_o - ref);
        m_run = m_new;
        l_run = l_run * fa + l_o * fb;
#pragma unroll
        for (int i = 0; i < 2 * NB2; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) o_acc[i][r] = o_acc[i][r] * fa + base[(4 * i + r) * 64] * fb;
        }
    };
    __syncthreads();                 // every wave is done with its tile: the memory changes hands
    if (wv >= 2) park(wv - 2);
    __syncthreads();
    if (wv < 2) take(wv);
    __syncthreads();
    if (wv == 1) park(0);
    __syncthreads();
    if (wv != 0) return;
    take(0);
    float l_tot = l_run + xor16(l_run);
    l_tot += xor32(l_tot);
    if (head >= heads) return;
    const float f = (gate ? gate[t * heads + head] : 1.0f) / l_tot;
    A* orow = out + ((int64_t)head * n_tok + t) * rank;
#pragma unroll
    for (int b2 = 0; b2 < NB2; ++b2) {
        {
#pragma unroll
            for (int r = 0; r < 4; ++r) {        // row i = 4 * quarter + r of the pair's blocks: columns 2 i (even) and 2 i + 1 (odd)
                const int c = 32 * b2 + 2 * (4 * quarter + r);
                *reinterpret_cast<uint32_t*>(orow + c) = la_pack2<A>(o_acc[2 * b2][r] * f, o_acc[2 * b2 + 1][r] * f);
            }
        }
    }
}

// ---- prefill: four query tokens of one sequence share every key tile -----------------------------------------------------
// Workgroup = tokens 4g .. 4g+3 of the step's token list, if they belong to one sequence (other groups return at once and
// are served by the kernel above, launched with skip_groups); wave w owns token 4g + w and all of its keys.  A tile's rows
// are fetched once for the four tokens -- each wave brings a quarter of the k-steps, one tile ahead, into the other of
// two LDS buffers -- so the cache is read a quarter as often, no merge is needed at the end, and the score product takes
// its A operand from LDS.  One barrier per tile.  The arithmetic per tile is the kernel's above.
template <typename A, int RKM>
__global__ __launch_bounds__(256, (RKM <= 8 ? 2 : 1)) void latent_attn_mfma_tile_kernel(
    const A* __restrict__ q, const A* __restrict__ cache, const int32_t* __restrict__ kv_indices, const int64_t* __restrict__ kv_start,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ tok_seq,
    const float* __restrict__ gate, A* __restrict__ out, int heads, int rank, int64_t n_tok, float scale) {
    extern __shared__ float lds[];
    constexpr int NB2 = RKM, MY = (RKM + 3) / 4;
    const int64_t t0 = (int64_t)blockIdx.x * 4;
    if (t0 + 3 >= n_tok) return;
    const int b = tok_seq[t0];
    if (tok_seq[t0 + 3] != b) return;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, l16 = lane & 15, quarter = lane >> 4;
    const int64_t t = t0 + wv;
    const int head = blockIdx.y * 16 + l16;
    const int64_t q0 = qo_indptr[b];
    const int64_t first = (int64_t)kv_len[b] - (qo_indptr[b + 1] - q0) - q0 + 1;      // keys of token t: first + t
    const int64_t n_keys = first + t, n_keys_max = first + t0 + 3;
    const int32_t* idx = kv_indices + kv_start[b];
    const int row_elems = rank + LA_PAD;
    uint16_t* buf0 = reinterpret_cast<uint16_t*>(lds);
    uint16_t* buf1 = buf0 + 16 * row_elems;

    nvx_u32x4 qb[RKM];
#pragma unroll
    for (int ks = 0; ks < RKM; ++ks) {
        qb[ks] = nvx_u32x4{0u, 0u, 0u, 0u};
        if (head < heads) qb[ks] = *reinterpret_cast<const nvx_u32x4*>(q + ((int64_t)head * n_tok + t) * rank + 32 * ks + 8 * quarter);
    }
    nvx_f32x4 o_acc[2 * NB2];
#pragma unroll
    for (int i = 0; i < 2 * NB2; ++i) o_acc[i] = nvx_f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    const int64_t n_tiles = (n_keys_max + 15) >> 4;
    nvx_u32x4 a_nxt[MY];
    auto slot_of = [&](int64_t j) {
        const int64_t key = j * 16 + l16;
        return idx[key < n_keys_max ? key : 0];
    };
    auto fetch = [&](int slot) {
        const A* row = cache + (int64_t)slot * rank;
#pragma unroll
        for (int i = 0; i < MY; ++i)
            if (wv + 4 * i < RKM) a_nxt[i] = *reinterpret_cast<const nvx_u32x4*>(row + 32 * (wv + 4 * i) + 8 * quarter);
    };
    auto park = [&](uint16_t* buf) {
#pragma unroll
        for (int i = 0; i < MY; ++i)
            if (wv + 4 * i < RKM) *reinterpret_cast<nvx_u32x4*>(buf + l16 * row_elems + 32 * (wv + 4 * i) + 8 * quarter) = a_nxt[i];
    };
    int slot_nxt = 0;
    fetch(slot_of(0));
    if (1 < n_tiles) slot_nxt = slot_of(1);
    park(buf0);
    __syncthreads();
    for (int64_t j = 0; j < n_tiles; ++j) {
        const uint16_t* tile = (j & 1) ? buf1 : buf0;
        if (j + 1 < n_tiles) fetch(slot_nxt);
        if (j + 2 < n_tiles) slot_nxt = slot_of(j + 2);
        if (j * 16 < n_keys) {                                   // (a last tile may hold only keys of the later tokens)
            nvx_f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < RKM; ++ks) {
                const nvx_u32x4 a = *reinterpret_cast<const nvx_u32x4*>(tile + l16 * row_elems + 32 * ks + 8 * quarter);
                sacc = la_mfma32<A>(a, qb[ks], sacc);
            }
            float sv[4], mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sv[r] = (j * 16 + 4 * quarter + r) < n_keys ? sacc[r] * scale : -INFINITY;
                mx = fmaxf(mx, sv[r]);
            }
            mx = fmaxf(mx, xor16(mx));
            mx = fmaxf(mx, xor32(mx));
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __expf(m_run - m_new);
            const bool rescale = __any(alpha != 1.0f);
            m_run = m_new;
            l_run *= alpha;
            float p[4], ph[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r] = __expf(sv[r] - m_new);
                l_run += p[r];
                ph[r] = la_round<A>(p[r]);
            }
            const uint2 p_hi = make_uint2(la_pack2<A>(ph[0], ph[1]), la_pack2<A>(ph[2], ph[3]));
            const uint2 p_lo = make_uint2(la_pack2<A>(p[0] - ph[0], p[1] - ph[1]), la_pack2<A>(p[2] - ph[2], p[3] - ph[3]));
            const uint32_t* tile32 = reinterpret_cast<const uint32_t*>(tile);
#pragma unroll
            for (int b2 = 0; b2 < NB2; ++b2) {
                uint32_t d[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) d[r] = tile32[((4 * quarter + r) * row_elems + 32 * b2) / 2 + l16];
                const uint2 even = make_uint2((d[0] & 0xffffu) | (d[1] << 16), (d[2] & 0xffffu) | (d[3] << 16));
                const uint2 odd = make_uint2((d[0] >> 16) | (d[1] & 0xffff0000u), (d[2] >> 16) | (d[3] & 0xffff0000u));
                if (rescale) {
                    o_acc[2 * b2] *= alpha;
                    o_acc[2 * b2 + 1] *= alpha;
                }
                o_acc[2 * b2] = la_mfma16<A>(even, p_hi, o_acc[2 * b2]);
                o_acc[2 * b2] = la_mfma16<A>(even, p_lo, o_acc[2 * b2]);
                o_acc[2 * b2 + 1] = la_mfma16<A>(odd, p_hi, o_acc[2 * b2 + 1]);
                o_acc[2 * b2 + 1] = la_mfma16<A>(odd, p_lo, o_acc[2 * b2 + 1]);
            }
        }
        if (j + 1 < n_tiles) park((j & 1) ? buf0 : buf1);        // the buffer whose readers passed the barrier before
        __syncthreads();
    }
    float l_tot = l_run + xor16(l_run);
    l_tot += xor32(l_tot);
    if (head >= heads) return;
    const float f = (gate ? gate[t * heads + head] : 1.0f) / l_tot;
    A* orow = out + ((int64_t)head * n_tok + t) * rank;
#pragma unroll
    for (int b2 = 0; b2 < NB2; ++b2) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int c = 32 * b2 + 2 * (4 * quarter + r);
            *reinterpret_cast<uint32_t*>(orow + c) = la_pack2<A>(o_acc[2 * b2][r] * f, o_acc[2 * b2 + 1][r] * f);
        }
    }
}

template <typename A>
static void launch_prep(const void* x, int64_t x_stride, const float* w_q, const float* w_kv, float eps, const int64_t* slots, void* cq,
                        void* cache, int64_t n_slots, float* gate, int64_t n_tok, int q_rank, int kv_rank, int heads, hipStream_t s) {
    hipLaunchKernelGGL(latent_prep_kernel<A>, dim3((unsigned)n_tok), dim3(256), 0, s, (const A*)x, x_stride, w_q, w_kv, eps, slots, (A*)cq,
                       (A*)cache, n_slots, gate, q_rank, kv_rank, heads);
}

template <typename A>
static void launch_attn(const void* q, const void* cache, const int32_t* kv_indices, const int64_t* kv_start, const int32_t* kv_len,
                        const int32_t* qo_indptr, const int32_t* tok_seq, const float* gate, void* out, int heads, int rank, int64_t n_tok,
                        float scale, hipStream_t s) {
    if constexpr (sizeof(A) == 2) {
        const int steps = rank / 32;
        const bool built = steps <= 8 || steps == 10 || steps == 12 || steps == 14 || steps == 16;     // the ranks the kernel is built for
        if (rank % 32 == 0 && built && nvx_aligned16(q) && nvx_aligned16(cache) && nvx_aligned16(out) && n_tok <= 0x7fffffff) {
            const size_t tiles = (size_t)4 * 16 * (rank + LA_PAD) * 2, merge = (size_t)2 * (8 * steps + 2) * 64 * 4;
            const size_t lds = tiles > merge ? tiles : merge;
            const dim3 grid((unsigned)n_tok, (unsigned)((heads + 15) / 16));
            // a ragged step: groups of four tokens inside one sequence go to the tile-sharing kernel, the rest stay here
            const int grouped = qo_indptr != nullptr && n_tok >= 4;
            const dim3 grid4((unsigned)(n_tok / 4), grid.y);
            const size_t lds4 = (size_t)2 * 16 * (rank + LA_PAD) * 2;
#define NVX_LA_MFMA(RKM)                                                                                                            \
    do {                                                                                                                            \
        if (grouped)                                                                                                                \
            hipLaunchKernelGGL((latent_attn_mfma_tile_kernel<A, RKM>), grid4, dim3(256), lds4, s, (const A*)q, (const A*)cache,       \
                               kv_indices, kv_start, kv_len, qo_indptr, tok_seq, gate, (A*)out, heads, rank, n_tok, scale);           \
        hipLaunchKernelGGL((latent_attn_mfma_kernel<A, RKM>), grid, dim3(256), lds, s, (const A*)q, (const A*)cache, kv_indices,      \
                           kv_start, kv_len, qo_indptr, tok_seq, gate, (A*)out, heads, rank, n_tok, scale, grouped);                 \
    } while (0)
            switch (steps) {
                case 1: NVX_LA_MFMA(1); break;
                case 2: NVX_LA_MFMA(2); break;
                case 3: NVX_LA_MFMA(3); break;
                case 4: NVX_LA_MFMA(4); break;
                case 5: NVX_LA_MFMA(5); break;
                case 6: NVX_LA_MFMA(6); break;
                case 7: NVX_LA_MFMA(7); break;
                case 8: NVX_LA_MFMA(8); break;
                case 10: NVX_LA_MFMA(10); break;
                case 12: NVX_LA_MFMA(12); break;
                case 14: NVX_LA_MFMA(14); break;
                default: NVX_LA_MFMA(16); break;
            }
#undef NVX_LA_MFMA
            return;
        }
    }
    constexpr int HG = 4;
    const size_t lds = (size_t)(HG * rank + LA_KT * HG + LA_KT + 4 * HG) * 4;
    hipLaunchKernelGGL((latent_attn_kernel<A, HG>), dim3((unsigned)n_tok, (unsigned)((heads + HG - 1) / HG)), dim3(256), lds, s,
                       (const A*)q, (const A*)cache, kv_indices, kv_start, kv_len, qo_indptr, tok_seq, gate, (A*)out, heads, rank, n_tok,
                       scale);
}

}  // namespace NVX_NS

using namespace NVX_NS;

#define NVX_FMT_DISPATCH(fmt, CALL)                                         \
    do {                                                                    \
        if ((fmt) == 0) { typedef __bf16 A_; CALL; }                        \
        else if ((fmt) == 1) { typedef _Float16 A_; CALL; }                 \
        else { typedef float A_; CALL; }                                    \
    } while (0)

extern "C" int nvx_latent_prep(const void* x, int64_t x_row_stride, int fmt, const float* w_q, const float* w_kv, float eps,
                               const int64_t* slots, void* cq, void* cache, int64_t n_slots, float* gate, int64_t n_tok, int64_t q_rank,
                               int64_t kv_rank, int64_t heads, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_latent_prep: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && q_rank > 0 && kv_rank > 0 && heads > 0 && n_slots >= 0 && q_rank + kv_rank + heads < (1 << 30) &&
                    x_row_stride >= q_rank + kv_rank + heads,
                NVX_EINVAL, "nvx_latent_prep: bad sizes");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && w_q && w_kv && slots && cq && cache && gate, NVX_EINVAL, "nvx_latent_prep: null pointer");
    NVX_FMT_DISPATCH(fmt, launch_prep<A_>(x, x_row_stride, w_q, w_kv, eps, slots, cq, cache, n_slots, gate, n_tok, (int)q_rank, (int)kv_rank,
                                          (int)heads, (hipStream_t)stream));
    return nvx_check_launch("nvx_latent_prep");
}

extern "C" int nvx_latent_rope_prep(const void* x, int64_t x_row_stride, int fmt, int64_t q_off, int64_t kv_off, int64_t g_off,
                                    const int64_t* positions, const double* freq, float mag, const float* w_kv, float eps,
                                    const int64_t* slots, void* q_out, void* cache, int64_t n_slots, int64_t row_len, float* gate,
                                    int64_t n_tok, int64_t heads, int64_t dim, int64_t rot, int64_t kv_rank, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_latent_rope_prep: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && heads > 0 && dim >= 0 && rot >= 0 && rot % 2 == 0 && rot <= 8192 && dim + rot > 0 && kv_rank > 0 && n_slots >= 0 &&
                    row_len >= kv_rank + rot && heads * (dim + rot) < (1 << 30) && row_len < (1 << 30),
                NVX_EINVAL, "nvx_latent_rope_prep: bad sizes (the rotated part is even, a cache row holds the latent and the rotated key part)");
    NVX_REQUIRE(q_off >= 0 && kv_off >= 0 && g_off >= 0 && x_row_stride >= q_off + heads * (dim + rot) && x_row_stride >= kv_off + kv_rank + rot &&
                    x_row_stride >= g_off + heads, NVX_EINVAL, "nvx_latent_rope_prep: a part lies outside a row");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && positions && (freq || rot == 0) && w_kv && slots && q_out && cache && gate, NVX_EINVAL, "nvx_latent_rope_prep: null pointer");
    NVX_FMT_DISPATCH(fmt, hipLaunchKernelGGL(latent_rope_prep_kernel<A_>, dim3((unsigned)n_tok), dim3(256), (size_t)(rot + 2) * sizeof(float),
                                             (hipStream_t)stream, (const A_*)x, x_row_stride, (int)q_off, (int)kv_off, (int)g_off, positions, freq,
                                             mag, w_kv, eps, slots, (A_*)q_out, (A_*)cache, n_slots, (int)row_len, gate, (int)heads, (int)dim,
                                             (int)rot, (int)kv_rank));
    return nvx_check_launch("nvx_latent_rope_prep");
}

extern "C" int nvx_latent_attn(const void* q, const void* cache, int fmt, const int32_t* kv_indices, const int64_t* kv_start,
                               const int32_t* kv_len, const int32_t* qo_indptr, const int32_t* tok_seq, const float* gate, void* out,
                               int64_t heads, int64_t rank, int64_t n_tok, float scale, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_latent_attn: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && heads > 0 && heads <= 65535 * 4 && rank > 0, NVX_EINVAL, "nvx_latent_attn: bad sizes");
    NVX_REQUIRE(rank <= 256 * LA_MAXC, NVX_EUNSUPPORTED, "nvx_latent_attn: latent size above 1024");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(q && cache && kv_indices && kv_start && kv_len && out, NVX_EINVAL, "nvx_latent_attn: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_latent_attn: tok_seq and qo_indptr go together");
    NVX_FMT_DISPATCH(fmt, launch_attn<A_>(q, cache, kv_indices, kv_start, kv_len, qo_indptr, tok_seq, gate, out, (int)heads, (int)rank, n_tok,
                                          scale, (hipStream_t)stream));
    return nvx_check_launch("nvx_latent_attn");
}
