// Causal attention over per-token key and value rows addressed through slot lists, for heads whose key size and value size
// differ, with grouped key/value heads, rotary positions on a leading part of each head (frequencies given as a table, so
// any scaling of them is the caller's), values scaled to unit mean square before they are cached, and scores that pass
// cap * tanh(score / cap) before the softmax.
//   - nvx_rope_vnorm_store: after the fused q|k|v projection: rotate q and k, norm v, scatter k and v into the caches;
//   - nvx_attn_prep_store: the same place for heads with a query/key RMS norm (per head, or over all heads of a row at once), a
//     rotation in either pair layout, and values that are themselves rotated by their position before they are cached;
//   - nvx_softcap_attn: the attention itself; scores, maxima, exponentials and sums are float32 in every format.  Optional: a
//     sliding window, a logarithmic distance penalty per head, a sink (one more term in the softmax's sum, with a score of its
//     own and no value), the read-out turned back by the query's position (the counterpart of rotated values) and multiplied by
//     a sigmoid gate (one per element, or one per head).
#include "fmt_dev.h"

namespace NVX_NS {

// One workgroup per token.  x[t] = [q (heads * dim) | k (kv_heads * dim) | v (kv_heads * vdim)].  The first rot_dims of a
// head are rotated in pairs (i, i + rot_dims / 2) by the angle positions[t] * freq[i] (the product and its cosine and sine
// are formed in double precision, so the table alone sets the accuracy), both cos and sin times `mag`.
template <typename A>
__global__ __launch_bounds__(256) void rope_vnorm_store_kernel(const A* __restrict__ x, int64_t x_stride, const int64_t* __restrict__ positions,
                                                              const double* __restrict__ freq, float mag, int rot_dims, float eps,
                                                              const int64_t* __restrict__ slots, A* __restrict__ q_out,
                                                              A* __restrict__ k_cache, A* __restrict__ v_cache, int heads, int kv_heads,
                                                              int dim, int vdim) {
    extern __shared__ float cs[];      // cos (half), sin (half)
    const int64_t t = blockIdx.x;
    const int half = rot_dims / 2;
    const double pos = (double)positions[t];
    for (int i = threadIdx.x; i < half; i += 256) {
        const double a = pos * freq[i];
        cs[i] = (float)(cos(a) * (double)mag);
        cs[half + i] = (float)(sin(a) * (double)mag);
    }
    __syncthreads();
    const A* row = x + t * x_stride;
    const int64_t slot = slots[t];
    const int nq = heads * dim, nk = kv_heads * dim;
    for (int idx = threadIdx.x; idx < nq + nk; idx += 256) {
        const int d = idx % dim;
        const float v = ld_f(row, idx);
        float o = v;
        if (d < half) o = v * cs[d] - ld_f(row, idx + half) * cs[half + d];
        else if (d < rot_dims) o = v * cs[d - half] + ld_f(row, idx - half) * cs[d];
        if (idx < nq) st_f(q_out, t * (int64_t)nq + idx, o);
        else if (slot >= 0) st_f(k_cache, slot * (int64_t)nk + (idx - nq), o);
    }
    if (slot < 0) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int g = wave; g < kv_heads; g += 4) {
        const A* v = row + nq + nk + g * vdim;
        float ss = 0.f;
        for (int e = lane; e < vdim; e += 64) { const float u = ld_f(v, e); ss += u * u; }
        const float rn = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
        for (int e = lane; e < vdim; e += 64) st_f(v_cache, slot * (int64_t)kv_heads * vdim + g * vdim + e, ld_f(v, e) * rn);
    }
}


// cos and sin of an angle given in double precision (position * frequency, exact to the table's accuracy at any position): the
// angle is brought into [-pi, pi] in double precision, where its float32 value is off by at most 2e-7, and the float32 functions
// take it from there.
__device__ __forceinline__ void turn_of(double a, float& c, float& s) {
    const double two_pi = 6.283185307179586476925286766559;
    const float r = (float)(a - two_pi * rint(a / two_pi));
    sincosf(r, &s, &c);
}

// One workgroup per token.  q, k and v are heads * dim, kv_heads * dim and kv_heads * vdim elements of row t of x, at q_off, k_off
// and v_off (kv_heads == 0: a layer that borrows another layer's keys and values prepares its queries only).
//   norm_mode 1: every query and key head is divided by its root mean square and multiplied by q_w / k_w (dim entries, shared by
//                the heads);  norm_mode 2: the whole query row (all heads at once) and the whole key row likewise, q_w / k_w having
//                heads * dim / kv_heads * dim entries;  0: no norm.
//   The first rot_dims of every q and k head are then turned in pairs by positions[t] * freq[m]: pair m is (m, m + rot_dims / 2), or
//   (2m, 2m + 1) if `interleaved`.  With vfreq, every value head is turned the same way over all of vdim by positions[t] * vfreq[m].
// Angles are formed and reduced in double precision, cosines and sines taken in float32 from the reduced angle; the norm is float32.  vcs_out (n_tok, vdim), if given, receives every
// token's cos | sin of positions[t] * vfreq[m] (vdim / 2 each).
template <typename A>
__global__ __launch_bounds__(256) void attn_prep_store_kernel(const A* __restrict__ x, int64_t x_stride, int q_off, int k_off, int v_off,
                                                             const int64_t* __restrict__ positions, const float* __restrict__ q_w,
                                                             const float* __restrict__ k_w, int norm_mode, float eps,
                                                             const double* __restrict__ freq, int rot_dims, int interleaved,
                                                             const double* __restrict__ vfreq, const int64_t* __restrict__ slots,
                                                             A* __restrict__ q_out, A* __restrict__ k_cache, A* __restrict__ v_cache, int heads,
                                                             int kv_heads, int dim, int vdim, float* __restrict__ vcs_out) {
    extern __shared__ float sm[];
    __shared__ float red[4];
    const int nq = heads * dim, nk = kv_heads * dim, nv = kv_heads * vdim;
    const int half = rot_dims / 2, vhalf = vdim / 2;
    float* buf = sm;                    // nq + nk: the query and key rows
    float* cs = buf + nq + nk;          // rot_dims: cos | sin
    float* vcs = cs + rot_dims;         // vdim (with vfreq): cos | sin
    const int64_t t = blockIdx.x;
    const double pos = (double)positions[t];
    const A* row = x + t * x_stride;
    for (int i = threadIdx.x; i < half; i += 256) turn_of(pos * freq[i], cs[i], cs[half + i]);
    if (vfreq)                          // also handed out (vcs_out[t] = cos | sin): the attention turns its read-out back by the same angles
        for (int i = threadIdx.x; i < vhalf; i += 256) {
            float cv, sv;
            turn_of(pos * vfreq[i], cv, sv);
            vcs[i] = cv;
            vcs[vhalf + i] = sv;
            if (vcs_out) { vcs_out[t * (int64_t)vdim + i] = cv; vcs_out[t * (int64_t)vdim + vhalf + i] = sv; }
        }
    for (int i = threadIdx.x; i < nq + nk; i += 256) buf[i] = ld_f(row, i < nq ? q_off + i : k_off + (i - nq));
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (norm_mode == 1) {
        for (int hh = wave; hh < heads + kv_heads; hh += 4) {
            float* r = buf + hh * dim;
            const float* w = hh < heads ? q_w : k_w;
            float ss = 0.f;
            for (int d = lane; d < dim; d += 64) ss += r[d] * r[d];
            const float rn = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
            for (int d = lane; d < dim; d += 64) r[d] = r[d] * rn * w[d];
        }
        __syncthreads();
    } else if (norm_mode == 2) {
        float a = 0.f, b = 0.f;
        for (int i = threadIdx.x; i < nq; i += 256) a += buf[i] * buf[i];
        for (int i = threadIdx.x; i < nk; i += 256) b += buf[nq + i] * buf[nq + i];
        const float rq = 1.0f / sqrtf(block256_sum(a, red) / (float)nq + eps);
        const float rk = nk ? 1.0f / sqrtf(block256_sum(b, red) / (float)nk + eps) : 0.f;
        for (int i = threadIdx.x; i < nq; i += 256) buf[i] = buf[i] * rq * q_w[i];
        for (int i = threadIdx.x; i < nk; i += 256) buf[nq + i] = buf[nq + i] * rk * k_w[i];
        __syncthreads();
    }
    const int64_t slot = slots ? slots[t] : -1;
    for (int idx = threadIdx.x; idx < nq + nk; idx += 256) {
        const int d = idx % dim;
        const float v = buf[idx];
        float o = v;
        if (d < rot_dims) {
            if (interleaved) {
                const int m = d >> 1;
                o = (d & 1) ? v * cs[m] + buf[idx - 1] * cs[half + m] : v * cs[m] - buf[idx + 1] * cs[half + m];
            } else {
                o = d < half ? v * cs[d] - buf[idx + half] * cs[half + d] : v * cs[d - half] + buf[idx - half] * cs[d];
            }
        }
        if (idx < nq) st_f(q_out, t * (int64_t)nq + idx, o);
        else if (slot >= 0) st_f(k_cache, slot * (int64_t)nk + (idx - nq), o);
    }
    if (slot < 0) return;
    const A* vr = row + v_off;
    for (int idx = threadIdx.x; idx < nv; idx += 256) {
        const int e = idx % vdim;
        const float v = ld_f(vr, idx);
        float o = v;
        if (vfreq) {
            if (interleaved) {
                const int m = e >> 1;
                o = (e & 1) ? v * vcs[m] + ld_f(vr, idx - 1) * vcs[vhalf + m] : v * vcs[m] - ld_f(vr, idx + 1) * vcs[vhalf + m];
            } else {
                o = e < vhalf ? v * vcs[e] - ld_f(vr, idx + vhalf) * vcs[vhalf + e] : v * vcs[e - vhalf] + ld_f(vr, idx - vhalf) * vcs[e];
            }
        }
        st_f(v_cache, slot * (int64_t)nv + idx, o);
    }
}

// The end of an attention read-out for one (token, head): `so` holds its vdim values in LDS (every thread of the workgroup has
// passed a barrier since they were written).  With `turn` (the query token's cos | sin row, vdim / 2 each, as nvx_attn_prep_store
// hands it out) the pairs are turned BACK by those angles (values were cached turned by their own positions, so the weighted sum
// is a sum of values in the query's frame); with a gate row every element is multiplied by sigmoid(gate): its own entry of the
// row, or the row's one entry for the whole head (`gate_one`).
template <typename A>
__device__ __forceinline__ void attn_readout_end(float* so, int vdim, const float* __restrict__ turn, int interleaved,
                                                 const A* __restrict__ gate_row, bool gate_one, A* __restrict__ out_row, int n_threads) {
    if (turn) {
        const int vhalf = vdim / 2;
        for (int m = threadIdx.x; m < vhalf; m += n_threads) {
            const int i0 = interleaved ? 2 * m : m, i1 = interleaved ? 2 * m + 1 : m + vhalf;
            const float c = turn[m], s = turn[vhalf + m];
            const float u = so[i0], v = so[i1];
            so[i0] = u * c + v * s;
            so[i1] = v * c - u * s;
        }
        __syncthreads();
    }
    for (int e = threadIdx.x; e < vdim; e += n_threads) {
        float v = so[e];
        if (gate_row) v *= sigmoid_f(ld_f(gate_row, gate_one ? 0 : e));
        st_f(out_row, e, v);
    }
}

__device__ __forceinline__ float lane_value(float v, int lane) {      // `lane` is the same in every lane of the wave
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// One workgroup of four waves per (head, token).  The waves take the visible keys in tiles of 64, every fourth tile each: a
// lane scores one key (the query waits in LDS), the wave keeps a running maximum and sum, then each lane accumulates the
// weighted values of EPL of the head's value columns over the tile's keys.  The four partial results are merged through LDS.
template <typename A, int EPL, bool VEC>
__global__ __launch_bounds__(256) void softcap_attn_kernel(const A* __restrict__ q, const A* __restrict__ k_cache, const A* __restrict__ v_cache,
                                                          const int32_t* __restrict__ kv_indices, const int64_t* __restrict__ kv_start,
                                                          const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr,
                                                          const int32_t* __restrict__ tok_seq, float scale, float cap, A* __restrict__ out,
                                                          int heads, int kv_heads, int dim, int vdim, int vec_v_ok, int n_split,
                                                          float* __restrict__ part, int window, const float* __restrict__ r1,
                                                          const float* __restrict__ r2, const float* __restrict__ vcs, int v_inter,
                                                          const A* __restrict__ gate, int64_t gate_stride, int gate_one, int sink,
                                                          float sink_score) {
    extern __shared__ float sm[];
    float* sq = sm;                   // dim
    float* sacc = sq + dim;           // 4 * vdim
    float* sml = sacc + 4 * vdim;     // 4 maxima, 4 sums
    const int hd = blockIdx.x;
    const int64_t t = blockIdx.y;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const int64_t q0 = qo_indptr ? qo_indptr[b] : b;
    const int64_t q_n = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
    const int visible = kv_len[b] - (int)(q_n - 1 - (t - q0));
    // a window of w keys: the token itself and the w - 1 before it
    const int first = (window > 0 && visible > window) ? visible - window : 0;
    const float pen_a = r1 ? r1[hd] : 0.f, pen_b = r1 ? r2[hd] : 0.f;
    const int kvh = hd / (heads / kv_heads);
    const int32_t* slots = kv_indices + kv_start[b];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int d = threadIdx.x; d < dim; d += 256) sq[d] = ld_f(q, t * (int64_t)heads * dim + (int64_t)hd * dim + d);
    __syncthreads();
    const int64_t k_row = (int64_t)kv_heads * dim, v_row = (int64_t)kv_heads * vdim;
    float m = -INFINITY, l = 0.f;
    float acc[EPL];
#pragma unroll
    for (int c = 0; c < EPL; ++c) acc[c] = 0.f;
    float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // value rows by 16-byte loads: vdim = 8 * (a power of two up to 64), rows 16-byte aligned (the caller checks the base)
    const bool vec_values = VEC && (vdim & 7) == 0 && ((vdim >> 3) & ((vdim >> 3) - 1)) == 0 && (vdim >> 3) <= 64 && vec_v_ok;
    // with n_split > 1 (steps of few tokens) the key tiles are dealt out over n_split workgroups as well as over the four waves
    for (int j0 = first + (blockIdx.z * 4 + wave) * 64; j0 < visible; j0 += 256 * n_split) {
        const int j = j0 + lane;
        const bool valid = j < visible;
        const int slot = valid ? slots[j] : 0;
        float s = -INFINITY;
        if (valid) {
            const A* kr = k_cache + slot * k_row + (int64_t)kvh * dim;
            float dot = 0.f;
            if constexpr (VEC) {          // 16-bit rows, 16-byte aligned, dim a multiple of 8: eight elements a load
                typedef A vec8 __attribute__((ext_vector_type(8)));
                for (int d = 0; d < dim; d += 8) {
                    const vec8 kv = *reinterpret_cast<const vec8*>(kr + d);
#pragma unroll
                    for (int i = 0; i < 8; ++i) dot += sq[d + i] * (float)kv[i];
                }
            } else {
                for (int d = 0; d < dim; ++d) dot += sq[d] * ld_f(kr, d);
            }
            s = dot * scale;
            if (cap > 0.f) s = cap * tanhf(s / cap);
            if (r1) s -= pen_a * log1pf(pen_b * (float)(visible - 1 - j));      // the penalty grows with the distance to the query
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float corr = expf(m - m_new);          // first tile: exp(-inf) = 0
        const float p = valid ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int c = 0; c < EPL; ++c) acc[c] *= corr;
        const int n_here = visible - j0 < 64 ? visible - j0 : 64;
        if constexpr (VEC) {
            // a value row is vdim / 8 lanes of eight elements (16-byte loads), so 64 / (vdim / 8) keys are taken at a time
            if (vec_values) {
                const int lpr = vdim >> 3, grp = lane / lpr, groups = 64 / lpr;
                typedef A vec8 __attribute__((ext_vector_type(8)));
#pragma unroll
                for (int i = 0; i < 8; ++i) acc8[i] *= corr;
                for (int j1 = 0; j1 < n_here; j1 += groups) {
                    const int jj = j1 + grp;
                    const int src = jj < n_here ? jj : 0;
                    const float pj = __shfl(p, src, 64);
                    const int sl = __shfl(slot, src, 64);
                    if (jj < n_here) {
                        const vec8 vv = *reinterpret_cast<const vec8*>(v_cache + sl * v_row + (int64_t)kvh * vdim + (lane % lpr) * 8);
#pragma unroll
                        for (int i = 0; i < 8; ++i) acc8[i] += pj * (float)vv[i];
                    }
                }
                continue;
            }
        }
        for (int jj = 0; jj < n_here; ++jj) {
            const float pj = lane_value(p, jj);
            const int sl = __builtin_amdgcn_readlane(slot, jj);
            const A* vr = v_cache + sl * v_row + (int64_t)kvh * vdim;
#pragma unroll
            for (int c = 0; c < EPL; ++c) {
                const int e = lane + 64 * c;
                if (e < vdim) acc[c] += pj * ld_f(vr, e);
            }
        }
    }
    if (VEC && vec_values) {
        const int lpr = vdim >> 3;
        for (int mk = lpr; mk < 64; mk <<= 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc8[i] += __shfl_xor(acc8[i], mk, 64);
        }
        if (lane < lpr) {
#pragma unroll
            for (int i = 0; i < 8; ++i) sacc[wave * vdim + lane * 8 + i] = acc8[i];
        }
    } else {
#pragma unroll
        for (int c = 0; c < EPL; ++c) {
            const int e = lane + 64 * c;
            if (e < vdim) sacc[wave * vdim + e] = acc[c];
        }
    }
    if (lane == 0) { sml[wave] = m; sml[4 + wave] = l; }
    __syncthreads();
    float* pr = n_split > 1 ? part + ((t * heads + hd) * (int64_t)n_split + blockIdx.z) * (vdim + 2) : nullptr;
    // a sink is one more term of the softmax's sum, with a score of its own and no value (a split's parts get it where they are merged)
    const bool sunk = sink && !pr;
    const float mm = fmaxf(fmaxf(fmaxf(sml[0], sml[1]), fmaxf(sml[2], sml[3])), sunk ? sink_score : -INFINITY);
    float f[4], total = sunk ? expf(sink_score - mm) : 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) { f[w] = sml[w] == -INFINITY ? 0.f : expf(sml[w] - mm); total += sml[4 + w] * f[w]; }
    for (int e = threadIdx.x; e < vdim; e += 256) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) o += sacc[w * vdim + e] * f[w];
        if (pr) pr[2 + e] = o;
        else if (vcs || gate) sacc[e] = o / total;            // (this thread alone reads column e of the four partial sums)
        else st_f(out, t * (int64_t)heads * vdim + (int64_t)hd * vdim + e, o / total);
    }
    if (pr && threadIdx.x == 0) { pr[0] = mm; pr[1] = total; }
    if (!pr && (vcs || gate)) {
        __syncthreads();
        attn_readout_end<A>(sacc, vdim, vcs ? vcs + t * (int64_t)vdim : nullptr, v_inter,
                            gate ? gate + t * gate_stride + (gate_one ? (int64_t)hd : (int64_t)hd * vdim) : nullptr, gate_one != 0,
                            out + t * (int64_t)heads * vdim + (int64_t)hd * vdim, 256);
    }
}

// ---- the same attention on the matrix cores, for steps of many tokens in a 16-bit format -------------------------------------
// A workgroup takes 64 consecutive query tokens of ONE sequence and one query head; each of its four waves owns 16 of them.  Keys
// are walked in tiles of 32.  Per tile and wave:
//   S^T (16 keys x 16 queries), twice = K_tile (16 x dim) . Q^T (dim x 16)      v_mfma_f32_16x16x32, dim / 32 of them each; the A
//       operand comes straight from the cache rows (lane (key, quarter) takes 16 bytes per step), fetched one tile ahead, the B
//       operand (the wave's queries) stays in registers;
//   the result leaves every lane with ONE query (lane & 15) and eight keys (4 * quarter + r of both halves): scale, cap, penalty,
//       mask, running maximum and sum are float32 per lane, reduced over the quarters by lane exchange;
//   O^T (vdim x 16 queries) += V_tile^T (vdim x 32 keys) . P^T (32 keys x 16 queries)      v_mfma_f32_16x16x32, vdim / 16 of them, twice:
//       the weights stay float32 up to here and enter as hi + lo, which keeps 16 bits of their mantissa; P^T is what the lane
//       holds (its eight keys in the order quarter-of-half-0, quarter-of-half-1), and V^T is read from an LDS tile in that same key
//       order; the tile is written transposed by the whole workgroup, once for its four waves.
// At the end a lane holds, for its query, value columns 16 * tile + 4 * quarter + r: both partners of a pair that is turned back
// (halves: tiles vt and vt + VT / 2; side by side: r and r + 1) are in the lane, so the read-out's end needs no exchange.
typedef __attribute__((ext_vector_type(8))) __bf16 ca_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 ca_f16x8;
template <typename A> __device__ __forceinline__ nvx_f32x4 ca_mfma32(nvx_u32x4 a, nvx_u32x4 b, nvx_f32x4 c) {
    if constexpr (__is_same(A, __bf16))
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(ca_bf16x8, a), __builtin_bit_cast(ca_bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(ca_f16x8, a), __builtin_bit_cast(ca_f16x8, b), c, 0, 0, 0);
}
template <typename A> __device__ __forceinline__ uint32_t ca_pack2(float lo, float hi) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    typedef A a2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, a2));
}

constexpr int TILE_Q = 64;       // query tokens per workgroup
constexpr int TILE_K = 32;       // keys per step
constexpr int VT_ROW = 40;       // elements per row of the V^T tile in LDS: 32 keys and a pad that spreads the rows over the banks

template <typename A, int DS, int VT>
__global__ __launch_bounds__(256) void softcap_attn_tile_kernel(const A* __restrict__ q, const A* __restrict__ k_cache, const A* __restrict__ v_cache,
                                                               const int32_t* __restrict__ kv_indices, const int64_t* __restrict__ kv_start,
                                                               const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr, int n_seq,
                                                               float scale, float cap, A* __restrict__ out, int heads, int kv_heads, int window,
                                                               const float* __restrict__ r1, const float* __restrict__ r2,
                                                               const float* __restrict__ vcs, int v_inter, const A* __restrict__ gate,
                                                               int64_t gate_stride, int gate_one, int sink, float sink_score) {
    constexpr int dim = DS * 32, vdim = VT * 16;
    __shared__ A vt_lds[vdim * VT_ROW];
    __shared__ int where[2];
    if (threadIdx.x == 0) {          // which sequence and which block of its tokens: sequences take ceil(tokens / 64) workgroups each
        // Workgroups start in the order of their numbers, and a block late in a portion has the most keys to walk: the count runs
        // backwards (last sequence first, and of a sequence its last block first), all heads of a block side by side, so the long
        // walks start first and the short ones fill the end.
        int rem = (int)(gridDim.y - 1 - blockIdx.y), found = -1;
        for (int b = n_seq - 1; b >= 0; --b) {
            const int nb = (qo_indptr[b + 1] - qo_indptr[b] + TILE_Q - 1) / TILE_Q;
            if (rem < nb) { found = b; rem = nb - 1 - rem; break; }
            rem -= nb;
        }
        where[0] = found;
        where[1] = rem;
    }
    __syncthreads();
    const int b = where[0];
    if (b < 0) return;               // (the grid is an upper bound)
    const int hd = blockIdx.x, kvh = hd / (heads / kv_heads);
    const int q0 = qo_indptr[b], q_n = qo_indptr[b + 1] - q0, qs = where[1] * TILE_Q;
    const int rows_here = q_n - qs < TILE_Q ? q_n - qs : TILE_Q;
    const int pos_first = kv_len[b] - q_n + qs;                 // position of the block's first query
    const int hi = pos_first + rows_here;                       // keys [lo, hi) are seen by some query of the block
    const int lo = window > 0 && pos_first - window + 1 > 0 ? pos_first - window + 1 : 0;
    const int32_t* slots = kv_indices + kv_start[b];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
    const int row = wave * 16 + c;
    const bool row_on = row < rows_here;
    const int pos = pos_first + row;
    const int w_hi = pos_first + wave * 16 + 16 < hi ? pos_first + wave * 16 + 16 : hi;      // this wave's queries see [w_lo, w_hi)
    const int w_lo = window > 0 && pos_first + wave * 16 - window + 1 > 0 ? pos_first + wave * 16 - window + 1 : 0;
    const bool wave_on = wave * 16 < rows_here;
    const int64_t k_row = (int64_t)kv_heads * dim, v_row = (int64_t)kv_heads * vdim;
    nvx_u32x4 qb[DS];
    {
        const A* qr = q + ((int64_t)q0 + qs + (row_on ? row : rows_here - 1)) * heads * dim + (int64_t)hd * dim + 8 * g;
#pragma unroll
        for (int s = 0; s < DS; ++s) qb[s] = *reinterpret_cast<const nvx_u32x4*>(qr + 32 * s);
    }
    const float pen_a = r1 ? r1[hd] : 0.f, pen_b = r1 ? r2[hd] : 0.f;
    nvx_f32x4 acc[VT];
#pragma unroll
    for (int t = 0; t < VT; ++t) acc[t] = nvx_f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    // Rows hang on slot ids, which hang on the slot list: two memory round trips in a row.  The ids are read two tiles ahead and the
    // rows one tile ahead (keys into the registers the products read, values into registers that the next step writes to LDS),
    // so that neither wait stands in front of a tile's products.
    constexpr int VCH = TILE_K * (vdim / 8);                         // 16-byte pieces of a tile of values
    constexpr int VPT = (VCH + 255) / 256;                           // ... per thread
    typedef A vec8 __attribute__((ext_vector_type(8)));
    nvx_u32x4 kf[2][DS];
    vec8 vf[VPT];
    int k_slot[2], v_slot[VPT];
    auto fetch_slots = [&](int j0) {                                 // (a key past the end reads a real row and is masked)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) { const int j = j0 + hh * 16 + c; k_slot[hh] = slots[j < hi ? j : hi - 1]; }
#pragma unroll
        for (int u = 0; u < VPT; ++u) { const int j = j0 + ((threadIdx.x + 256 * u) & (TILE_K - 1)); v_slot[u] = slots[j < hi ? j : hi - 1]; }
    };
    auto fetch_key_rows = [&]() {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const A* kr = k_cache + (int64_t)k_slot[hh] * k_row + (int64_t)kvh * dim + 8 * g;
#pragma unroll
            for (int s = 0; s < DS; ++s) kf[hh][s] = *reinterpret_cast<const nvx_u32x4*>(kr + 32 * s);
        }
    };
    auto fetch_value_rows = [&]() {
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (i < VCH) vf[u] = *reinterpret_cast<const vec8*>(v_cache + (int64_t)v_slot[u] * v_row + (int64_t)kvh * vdim + (i / TILE_K) * 8);
        }
    };
    // Scores live in the log2 domain (the hardware's exponential and logarithm are base 2): s2 = log2(e) * score.
    //   no cap:  s2 = acc * (scale log2 e);   cap:  tanh(x) = 1 - 2 / (e^(2x) + 1), so s2 = (cap log2 e) (1 - 2 / (2^(acc * 2 scale log2 e / cap) + 1));
    //   penalty: s2 -= r1 log2(1 + r2 distance).
    constexpr float LOG2E = 1.4426950408889634f;
    const float k_lin = cap > 0.f ? 2.0f * scale * LOG2E / cap : scale * LOG2E, k_cap = cap * LOG2E;
    const int j_begin = lo & ~(TILE_K - 1);
    fetch_slots(j_begin);
    if (wave_on) fetch_key_rows();
    fetch_value_rows();
    if (j_begin + TILE_K < hi) fetch_slots(j_begin + TILE_K);
    const int q_lo = pos_first + wave * 16;                          // positions of this wave's first and last query
    const int q_hi = q_lo + 15;
    const bool rows_full = wave * 16 + 16 <= rows_here;
    for (int j0 = j_begin; j0 < hi; j0 += TILE_K) {
        __syncthreads();                                             // the tile before has been read by all waves
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (i < VCH) {
                const int kk = i & (TILE_K - 1), ch = i / TILE_K;
#pragma unroll
                for (int e = 0; e < 8; ++e) vt_lds[(ch * 8 + e) * VT_ROW + kk] = vf[u][e];
            }
        }
        __syncthreads();
        // issued behind the barrier (which waits for every load before it): the next tile's rows and the ids of the one after
        // travel while this tile's products run; the key rows as soon as this tile's have been multiplied
        const bool more = j0 + TILE_K < hi;
        if (more) fetch_value_rows();                                // (with the ids read one step ago)
        if (!wave_on) {
            if (j0 + 2 * TILE_K < hi) fetch_slots(j0 + 2 * TILE_K);
            continue;
        }
        const bool seen = j0 < w_hi && j0 + TILE_K > w_lo;           // some query of this wave sees some key of the tile
        nvx_f32x4 sacc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        if (seen) {
#pragma unroll
            for (int s = 0; s < DS; ++s) {
                sacc[0] = ca_mfma32<A>(kf[0][s], qb[s], sacc[0]);
                sacc[1] = ca_mfma32<A>(kf[1][s], qb[s], sacc[1]);
            }
        }
        if (more) fetch_key_rows();
        if (j0 + 2 * TILE_K < hi) fetch_slots(j0 + 2 * TILE_K);
        if (!seen) continue;
        // every query of the wave sees every key of the tile (most tiles): no mask to work out
        const bool full = rows_full && j0 + TILE_K - 1 <= q_lo && (window <= 0 || j0 > q_hi - window);
        float sv[8], mx = -INFINITY;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = j0 + hh * 16 + 4 * g + r;
                float sc = sacc[hh][r] * k_lin;
                if (cap > 0.f) sc = k_cap - 2.0f * k_cap * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(sc) + 1.0f);
                if (r1) sc -= pen_a * __builtin_amdgcn_logf(1.0f + pen_b * (float)(pos - j));
                if (!full && !(row_on && j <= pos && (window <= 0 || j > pos - window))) sc = -INFINITY;
                sv[hh * 4 + r] = sc;
                mx = fmaxf(mx, sc);
            }
        }
        mx = fmaxf(mx, xor16(mx));
        mx = fmaxf(mx, xor32(mx));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);    // (nothing seen yet: nothing to rescale)
        m_run = m_new;
        l_run *= alpha;
        const float m_sub = m_new == -INFINITY ? 0.f : m_new;        // (then every score is -inf and every weight 0)
        float p[8], ph[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            p[e] = __builtin_amdgcn_exp2f(sv[e] - m_sub);
            l_run += p[e];
            ph[e] = (float)(A)p[e];
        }
        const nvx_u32x4 p_hi = {ca_pack2<A>(ph[0], ph[1]), ca_pack2<A>(ph[2], ph[3]), ca_pack2<A>(ph[4], ph[5]), ca_pack2<A>(ph[6], ph[7])};
        const nvx_u32x4 p_lo = {ca_pack2<A>(p[0] - ph[0], p[1] - ph[1]), ca_pack2<A>(p[2] - ph[2], p[3] - ph[3]),
                                ca_pack2<A>(p[4] - ph[4], p[5] - ph[5]), ca_pack2<A>(p[6] - ph[6], p[7] - ph[7])};
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int t = 0; t < VT; ++t) acc[t] *= alpha;
        }
#pragma unroll
        for (int t = 0; t < VT; ++t) {
            // row (value column) 16 t + c of V^T, keys 4 g .. 4 g + 3 of both halves: the order of the lane's weights
            const A* vr = vt_lds + (t * 16 + c) * VT_ROW + 4 * g;
            const uint2 a0 = *reinterpret_cast<const uint2*>(vr), a1 = *reinterpret_cast<const uint2*>(vr + 16);
            const nvx_u32x4 vfrag = {a0.x, a0.y, a1.x, a1.y};
            acc[t] = ca_mfma32<A>(vfrag, p_hi, acc[t]);
            acc[t] = ca_mfma32<A>(vfrag, p_lo, acc[t]);
        }
    }
    if (!wave_on) return;
    l_run += xor16(l_run);
    l_run += xor32(l_run);
    if (!row_on) return;
    if (sink) {                                                      // one more term of the sum, no value: the maximum may move to it
        const float s2 = sink_score * LOG2E, m_new = fmaxf(m_run, s2);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run = l_run * alpha + __builtin_amdgcn_exp2f(s2 - m_new);
#pragma unroll
        for (int t = 0; t < VT; ++t) acc[t] *= alpha;
    }
    const float inv = 1.0f / l_run;
#pragma unroll
    for (int t = 0; t < VT; ++t) acc[t] *= inv;
    const int64_t tok = (int64_t)q0 + qs + row;
    if (vcs) {
        const float* cs = vcs + tok * vdim, *sn = cs + vdim / 2;
        if (v_inter) {
#pragma unroll
            for (int t = 0; t < VT; ++t)
#pragma unroll
                for (int r = 0; r < 4; r += 2) {
                    const int m = (t * 16 + 4 * g + r) >> 1;
                    const float u = acc[t][r], v = acc[t][r + 1];
                    acc[t][r] = u * cs[m] + v * sn[m];
                    acc[t][r + 1] = v * cs[m] - u * sn[m];
                }
        } else {
#pragma unroll
            for (int t = 0; t < VT / 2; ++t) {
                const nvx_f32x4 c4 = *reinterpret_cast<const nvx_f32x4*>(cs + t * 16 + 4 * g), s4 = *reinterpret_cast<const nvx_f32x4*>(sn + t * 16 + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float u = acc[t][r], v = acc[t + VT / 2][r];
                    acc[t][r] = u * c4[r] + v * s4[r];
                    acc[t + VT / 2][r] = v * c4[r] - u * s4[r];
                }
            }
        }
    }
    A* orow = out + tok * heads * vdim + (int64_t)hd * vdim + 4 * g;
    const A* grow = gate && !gate_one ? gate + tok * gate_stride + (int64_t)hd * vdim + 4 * g : nullptr;
    const float g_head = gate && gate_one ? sigmoid_f((float)gate[tok * gate_stride + hd]) : 1.0f;      // one gate for the whole head
#pragma unroll
    for (int t = 0; t < VT; ++t) {
        float o[4] = {acc[t][0] * g_head, acc[t][1] * g_head, acc[t][2] * g_head, acc[t][3] * g_head};
        if (grow) {
            typedef A vec4 __attribute__((ext_vector_type(4)));
            const vec4 gv = *reinterpret_cast<const vec4*>(grow + t * 16);
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] *= sigmoid_f((float)gv[r]);
        }
        *reinterpret_cast<uint2*>(orow + t * 16) = make_uint2(ca_pack2<A>(o[0], o[1]), ca_pack2<A>(o[2], o[3]));
    }
}

// out = the n_split partial results of a (token, head) merged: each is (maximum, sum, unnormalised values); one wave each.
template <typename A>
__global__ __launch_bounds__(64) void softcap_merge_kernel(const float* __restrict__ part, int n_split, A* __restrict__ out, int vdim,
                                                          int heads, const float* __restrict__ vcs, int v_inter,
                                                          const A* __restrict__ gate, int64_t gate_stride, int gate_one, int sink,
                                                          float sink_score) {
    __shared__ float so[512];
    const int64_t row = blockIdx.x;
    const float* pr = part + row * n_split * (vdim + 2);
    float mm = sink ? sink_score : -INFINITY;
    for (int s = 0; s < n_split; ++s) mm = fmaxf(mm, pr[s * (vdim + 2)]);
    float total = sink ? expf(sink_score - mm) : 0.f;
    for (int s = 0; s < n_split; ++s) {
        const float m = pr[s * (vdim + 2)];
        total += m == -INFINITY ? 0.f : pr[s * (vdim + 2) + 1] * expf(m - mm);
    }
    for (int e = threadIdx.x; e < vdim; e += 64) {
        float o = 0.f;
        for (int s = 0; s < n_split; ++s) {
            const float m = pr[s * (vdim + 2)];
            if (m != -INFINITY) o += pr[s * (vdim + 2) + 2 + e] * expf(m - mm);
        }
        if (vcs || gate) so[e] = o / total;
        else st_f(out, row * vdim + e, o / total);
    }
    if (vcs || gate) {
        const int64_t t = row / heads;
        __syncthreads();
        attn_readout_end<A>(so, vdim, vcs ? vcs + t * (int64_t)vdim : nullptr, v_inter,
                            gate ? gate + t * gate_stride + (gate_one ? row % heads : (row % heads) * vdim) : nullptr, gate_one != 0,
                            out + row * vdim, 64);
    }
}

}  // namespace NVX_NS

using namespace NVX_NS;

// the tile kernel is built for 16-bit formats only; float stands in so that the format dispatch compiles (never launched)
template <typename T> struct tile_fmt { typedef T type; };
template <> struct tile_fmt<float> { typedef __bf16 type; };

// Whether nvx_softcap_attn has a matrix-core form for these sizes: 16-bit formats, key and value sizes of 64, 96 or 128; a read-out
// that is turned back in the halves layout needs both halves in whole column tiles.
extern "C" int nvx_softcap_attn_tile_fits(int fmt, int64_t dim, int64_t vdim, int turned_halves) {
    const bool sizes = (dim == 64 || dim == 96 || dim == 128) && (vdim == 64 || vdim == 96 || vdim == 128);
    return (fmt == 0 || fmt == 1) && sizes && (!turned_halves || (vdim / 16) % 2 == 0);
}

extern "C" int nvx_rope_vnorm_store(const void* x, int64_t x_stride, int fmt, const int64_t* positions, const double* freq, float mag,
                                    int rot_dims, float eps, const int64_t* slots, void* q_out, void* k_cache, void* v_cache,
                                    int64_t n_slots, int64_t n_tok, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                                    nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_rope_vnorm_store: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && n_slots >= 0 && (heads + kv_heads) * dim < (1 << 30) &&
                    kv_heads * vdim < (1 << 30), NVX_EINVAL, "nvx_rope_vnorm_store: bad sizes");
    NVX_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim && rot_dims <= 8192, NVX_EINVAL,
                "nvx_rope_vnorm_store: the rotated part must be even and within a head");
    NVX_REQUIRE(x_stride >= (heads + kv_heads) * dim + kv_heads * vdim, NVX_EINVAL, "nvx_rope_vnorm_store: row stride");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && positions && (freq || rot_dims == 0) && slots && q_out && k_cache && v_cache, NVX_EINVAL, "nvx_rope_vnorm_store: null pointer");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(rope_vnorm_store_kernel<A_>, dim3((unsigned)n_tok), dim3(256), (size_t)(rot_dims + 2) * sizeof(float),
                                         (hipStream_t)stream, (const A_*)x, x_stride, positions, freq, mag, rot_dims, eps, slots, (A_*)q_out,
                                         (A_*)k_cache, (A_*)v_cache, (int)heads, (int)kv_heads, (int)dim, (int)vdim));
    return nvx_check_launch("nvx_rope_vnorm_store");
}

extern "C" int nvx_attn_prep_store(const void* x, int64_t x_stride, int fmt, int64_t q_off, int64_t k_off, int64_t v_off,
                                   const int64_t* positions, const float* q_w, const float* k_w, int norm_mode, float eps, const double* freq,
                                   int rot_dims, int interleaved, const double* vfreq, const int64_t* slots, void* q_out, void* k_cache,
                                   void* v_cache, int64_t n_slots, int64_t n_tok, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                                   float* vcs_out, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && norm_mode >= 0 && norm_mode <= 2, NVX_EINVAL, "nvx_attn_prep_store: fmt must be 0..2, norm_mode 0..2");
    NVX_REQUIRE(n_tok >= 0 && heads > 0 && kv_heads >= 0 && dim > 0 && vdim > 0 && n_slots >= 0, NVX_EINVAL, "nvx_attn_prep_store: bad sizes");
    const int64_t nq = heads * dim, nk = kv_heads * dim, nv = kv_heads * vdim;
    NVX_REQUIRE(nq + nk + rot_dims + vdim <= 15360, NVX_EUNSUPPORTED, "nvx_attn_prep_store: a token's query and key rows must fit LDS as float32");
    NVX_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim && (rot_dims == 0 || freq), NVX_EINVAL,
                "nvx_attn_prep_store: the rotated part must be even and within a head");
    NVX_REQUIRE(!vfreq || vdim % 2 == 0, NVX_EINVAL, "nvx_attn_prep_store: rotated values have an even size");
    NVX_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && x_stride >= q_off + nq && (kv_heads == 0 || (x_stride >= k_off + nk && x_stride >= v_off + nv)),
                NVX_EINVAL, "nvx_attn_prep_store: q, k or v lies outside a row");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && positions && q_out && (norm_mode == 0 || (q_w && (k_w || kv_heads == 0))), NVX_EINVAL, "nvx_attn_prep_store: null pointer");
    NVX_REQUIRE(kv_heads == 0 || (slots && k_cache && v_cache), NVX_EINVAL, "nvx_attn_prep_store: keys and values need their caches and slots");
    const size_t lds = (size_t)(nq + nk + rot_dims + vdim) * sizeof(float);
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(attn_prep_store_kernel<A_>, dim3((unsigned)n_tok), dim3(256), lds, (hipStream_t)stream, (const A_*)x, x_stride,
                                         (int)q_off, (int)k_off, (int)v_off, positions, q_w, k_w, norm_mode, eps, freq, rot_dims, interleaved, vfreq,
                                         kv_heads ? slots : nullptr, (A_*)q_out, (A_*)k_cache, (A_*)v_cache, (int)heads, (int)kv_heads, (int)dim,
                                         (int)vdim, vcs_out));
    return nvx_check_launch("nvx_attn_prep_store");
}

extern "C" int nvx_softcap_attn(const void* q, const void* k_cache, const void* v_cache, int fmt, const int32_t* kv_indices,
                                const int64_t* kv_start, const int32_t* kv_len, const int32_t* qo_indptr, const int32_t* tok_seq,
                                float scale, float cap, void* out, int64_t n_tok, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                                int n_split, float* part, int64_t window, const float* r1, const float* r2, const float* vcs,
                                int v_interleaved, const void* gate, int64_t gate_stride, int gate_per_head, int sink, float sink_score,
                                int64_t n_seq, int matrix_cores, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_softcap_attn: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_tok <= 65535 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 4096 && vdim > 0 && vdim <= 512,
                NVX_EINVAL, "nvx_softcap_attn: bad sizes (at most 65535 tokens a step, key size <= 4096, value size <= 512)");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(q && k_cache && v_cache && kv_indices && kv_start && kv_len && out, NVX_EINVAL, "nvx_softcap_attn: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_softcap_attn: tok_seq and qo_indptr go together");
    NVX_REQUIRE((r1 != nullptr) == (r2 != nullptr), NVX_EINVAL, "nvx_softcap_attn: the distance penalty takes both of its numbers per head");
    NVX_REQUIRE(window >= 0 && window < (1ll << 31), NVX_EINVAL, "nvx_softcap_attn: bad window");
    NVX_REQUIRE(!vcs || (vdim % 2 == 0 && nvx_aligned16(vcs)), NVX_EINVAL, "nvx_softcap_attn: a read-out that is turned back has an even size");
    NVX_REQUIRE(!gate || gate_stride >= (gate_per_head ? heads : heads * vdim), NVX_EINVAL, "nvx_softcap_attn: row stride of the gate");
    // steps of many tokens in a 16-bit format, sizes the tile kernel is built for, 8-byte rows of the gate: the matrix cores
    if (matrix_cores && nvx_softcap_attn_tile_fits(fmt, dim, vdim, vcs != nullptr && !v_interleaved) && qo_indptr && n_split == 1 && n_seq > 0 &&
        nvx_aligned16(q) && nvx_aligned16(k_cache) && nvx_aligned16(v_cache) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0 &&
        (!gate || gate_per_head || ((reinterpret_cast<uintptr_t>(gate) & 7u) == 0 && gate_stride % 4 == 0))) {
        NVX_REQUIRE((n_tok + TILE_Q - 1) / TILE_Q + n_seq <= 65535, NVX_EINVAL, "nvx_softcap_attn: too many tokens or sequences in one step");
        const dim3 tgrid((unsigned)heads, (unsigned)((n_tok + TILE_Q - 1) / TILE_Q + n_seq));
#define NVX_TILE_ATTN(DS, VT)                                                                                                            \
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL((softcap_attn_tile_kernel<typename tile_fmt<A_>::type, DS, VT>), tgrid, dim3(256), 0, (hipStream_t)stream, \
                                         (const typename tile_fmt<A_>::type*)q, (const typename tile_fmt<A_>::type*)k_cache,            \
                                         (const typename tile_fmt<A_>::type*)v_cache, kv_indices, kv_start, kv_len, qo_indptr, (int)n_seq, scale, \
                                         cap, (typename tile_fmt<A_>::type*)out, (int)heads, (int)kv_heads, (int)window, r1, r2, vcs,    \
                                         v_interleaved, (const typename tile_fmt<A_>::type*)gate, gate_stride, gate_per_head, sink,   \
                                         sink_score))
#define NVX_TILE_ATTN_V(DS)                                                       \
    do {                                                                          \
        if (vdim == 64) NVX_TILE_ATTN(DS, 4);                                     \
        else if (vdim == 96) NVX_TILE_ATTN(DS, 6);                                \
        else NVX_TILE_ATTN(DS, 8);                                                \
    } while (0)
        if (dim == 64) NVX_TILE_ATTN_V(2);
        else if (dim == 96) NVX_TILE_ATTN_V(3);
        else NVX_TILE_ATTN_V(4);
#undef NVX_TILE_ATTN_V
#undef NVX_TILE_ATTN
        return nvx_check_launch("nvx_softcap_attn");
    }
    const size_t lds = (size_t)(dim + 4 * vdim + 8) * sizeof(float);
    NVX_REQUIRE(n_split >= 1 && n_split <= 64 && (n_split == 1 || part), NVX_EINVAL, "nvx_softcap_attn: a key split needs its workspace");
    const dim3 grid((unsigned)heads, (unsigned)n_tok, (unsigned)n_split);
#define NVX_CAP_ATTN_V(EPL, VEC)                                                                                                          \
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL((softcap_attn_kernel<A_, EPL, VEC && sizeof(A_) == 2>), grid, dim3(256), lds, (hipStream_t)stream,     \
                                         (const A_*)q, (const A_*)k_cache, (const A_*)v_cache, kv_indices, kv_start, kv_len, qo_indptr,      \
                                         tok_seq, scale, cap, (A_*)out, (int)heads, (int)kv_heads, (int)dim, (int)vdim,       \
                                         (int)nvx_aligned16(v_cache), n_split, part, (int)window, r1, r2, vcs, v_interleaved,   \
                                         (const A_*)gate, gate_stride, gate_per_head, sink, sink_score))
#define NVX_CAP_ATTN(EPL) do { if (vec) NVX_CAP_ATTN_V(EPL, true); else NVX_CAP_ATTN_V(EPL, false); } while (0)
    const bool vec = fmt != 2 && dim % 8 == 0 && nvx_aligned16(k_cache);
    if (vdim <= 64) NVX_CAP_ATTN(1);
    else if (vdim <= 128) NVX_CAP_ATTN(2);
    else if (vdim <= 256) NVX_CAP_ATTN(4);
    else NVX_CAP_ATTN(8);
#undef NVX_CAP_ATTN_V
    if (n_split > 1)
        NVX_FMT_CALL(fmt, hipLaunchKernelGGL(softcap_merge_kernel<A_>, dim3((unsigned)(n_tok * heads)), dim3(64), 0, (hipStream_t)stream,
                                             (const float*)part, n_split, (A_*)out, (int)vdim, (int)heads, vcs, v_interleaved, (const A_*)gate,
                                             gate_stride, gate_per_head, sink, sink_score));
#undef NVX_CAP_ATTN
    return nvx_check_launch("nvx_softcap_attn");
}
