// Causal attention over per-token key and value rows addressed through slot lists, for heads whose key size and value size
// differ, with grouped key/value heads, rotary positions on a leading part of each head (frequencies given as a table, so
// any scaling of them is the caller's), values scaled to unit mean square before they are cached, and scores that pass
// cap * tanh(score / cap) before the softmax.
//   - nvx_rope_vnorm_store: after the fused q|k|v projection: rotate q and k, norm v, scatter k and v into the caches;
//   - nvx_attn_prep_store: the same place for heads with a query/key RMS norm (per head, or over all heads of a row at once), a
//     rotation in either pair layout, and values that are themselves rotated by their position before they are cached;
//   - nvx_softcap_attn: the attention itself; scores, maxima, exponentials and sums are float32 in every format.  Optional: a
//     sliding window, a logarithmic distance penalty per head, the read-out turned back by the query's position (the
//     counterpart of rotated values) and multiplied by a sigmoid gate.
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


// One workgroup per token.  q, k and v are heads * dim, kv_heads * dim and kv_heads * vdim elements of row t of x, at q_off, k_off
// and v_off (kv_heads == 0: a layer that borrows another layer's keys and values prepares its queries only).
//   norm_mode 1: every query and key head is divided by its root mean square and multiplied by q_w / k_w (dim entries, shared by
//                the heads);  norm_mode 2: the whole query row (all heads at once) and the whole key row likewise, q_w / k_w having
//                heads * dim / kv_heads * dim entries;  0: no norm.
//   The first rot_dims of every q and k head are then turned in pairs by positions[t] * freq[m]: pair m is (m, m + rot_dims / 2), or
//   (2m, 2m + 1) if `interleaved`.  With vfreq, every value head is turned the same way over all of vdim by positions[t] * vfreq[m].
// Angles, cosines and sines are formed in double precision; the norm is float32.
template <typename A>
__global__ __launch_bounds__(256) void attn_prep_store_kernel(const A* __restrict__ x, int64_t x_stride, int q_off, int k_off, int v_off,
                                                             const int64_t* __restrict__ positions, const float* __restrict__ q_w,
                                                             const float* __restrict__ k_w, int norm_mode, float eps,
                                                             const double* __restrict__ freq, int rot_dims, int interleaved,
                                                             const double* __restrict__ vfreq, const int64_t* __restrict__ slots,
                                                             A* __restrict__ q_out, A* __restrict__ k_cache, A* __restrict__ v_cache, int heads,
                                                             int kv_heads, int dim, int vdim) {
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
    for (int i = threadIdx.x; i < half; i += 256) {
        const double a = pos * freq[i];
        cs[i] = (float)cos(a);
        cs[half + i] = (float)sin(a);
    }
    if (vfreq && nv)
        for (int i = threadIdx.x; i < vhalf; i += 256) {
            const double a = pos * vfreq[i];
            vcs[i] = (float)cos(a);
            vcs[vhalf + i] = (float)sin(a);
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
// passed a barrier since they were written).  With vfreq the pairs are turned BACK by pos * vfreq[m] (values were cached turned
// by their own positions, so the weighted sum is a sum of values in the query's frame); with a gate row every element is
// multiplied by sigmoid(gate).
template <typename A>
__device__ __forceinline__ void attn_readout_end(float* so, int vdim, int64_t pos, const double* __restrict__ vfreq, int interleaved,
                                                 const A* __restrict__ gate_row, A* __restrict__ out_row, int n_threads) {
    if (vfreq) {
        const int vhalf = vdim / 2;
        for (int m = threadIdx.x; m < vhalf; m += n_threads) {
            const int i0 = interleaved ? 2 * m : m, i1 = interleaved ? 2 * m + 1 : m + vhalf;
            const double a = (double)pos * vfreq[m];
            const float c = (float)cos(a), s = (float)sin(a);
            const float u = so[i0], v = so[i1];
            so[i0] = u * c + v * s;
            so[i1] = v * c - u * s;
        }
        __syncthreads();
    }
    for (int e = threadIdx.x; e < vdim; e += n_threads) {
        float v = so[e];
        if (gate_row) v *= sigmoid_f(ld_f(gate_row, e));
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
                                                          const float* __restrict__ r2, const double* __restrict__ vfreq, int v_inter,
                                                          const A* __restrict__ gate, int64_t gate_stride) {
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
    const float mm = fmaxf(fmaxf(sml[0], sml[1]), fmaxf(sml[2], sml[3]));
    float f[4], total = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) { f[w] = sml[w] == -INFINITY ? 0.f : expf(sml[w] - mm); total += sml[4 + w] * f[w]; }
    float* pr = n_split > 1 ? part + ((t * heads + hd) * (int64_t)n_split + blockIdx.z) * (vdim + 2) : nullptr;
    for (int e = threadIdx.x; e < vdim; e += 256) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) o += sacc[w * vdim + e] * f[w];
        if (pr) pr[2 + e] = o;
        else if (vfreq || gate) sacc[e] = o / total;          // (this thread alone reads column e of the four partial sums)
        else st_f(out, t * (int64_t)heads * vdim + (int64_t)hd * vdim + e, o / total);
    }
    if (pr && threadIdx.x == 0) { pr[0] = mm; pr[1] = total; }
    if (!pr && (vfreq || gate)) {
        __syncthreads();
        attn_readout_end<A>(sacc, vdim, visible - 1, vfreq, v_inter, gate ? gate + t * gate_stride + (int64_t)hd * vdim : nullptr,
                            out + t * (int64_t)heads * vdim + (int64_t)hd * vdim, 256);
    }
}

// out = the n_split partial results of a (token, head) merged: each is (maximum, sum, unnormalised values); one wave each.
template <typename A>
__global__ __launch_bounds__(64) void softcap_merge_kernel(const float* __restrict__ part, int n_split, A* __restrict__ out, int vdim,
                                                          int heads, const int32_t* __restrict__ kv_len, const int32_t* __restrict__ qo_indptr,
                                                          const int32_t* __restrict__ tok_seq, const double* __restrict__ vfreq, int v_inter,
                                                          const A* __restrict__ gate, int64_t gate_stride) {
    __shared__ float so[512];
    const int64_t row = blockIdx.x;
    const float* pr = part + row * n_split * (vdim + 2);
    float mm = -INFINITY;
    for (int s = 0; s < n_split; ++s) mm = fmaxf(mm, pr[s * (vdim + 2)]);
    float total = 0.f;
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
        if (vfreq || gate) so[e] = o / total;
        else st_f(out, row * vdim + e, o / total);
    }
    if (vfreq || gate) {
        const int64_t t = row / heads;
        const int b = tok_seq ? tok_seq[t] : (int)t;
        const int64_t q0 = qo_indptr ? qo_indptr[b] : b;
        const int64_t q_n = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
        const int64_t pos = kv_len[b] - (q_n - 1 - (t - q0)) - 1;
        __syncthreads();
        attn_readout_end<A>(so, vdim, pos, vfreq, v_inter, gate ? gate + t * gate_stride + (row % heads) * vdim : nullptr, out + row * vdim, 64);
    }
}

}  // namespace NVX_NS

using namespace NVX_NS;

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
                                   nvx_stream_t stream) {
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
                                         (int)vdim));
    return nvx_check_launch("nvx_attn_prep_store");
}

extern "C" int nvx_softcap_attn(const void* q, const void* k_cache, const void* v_cache, int fmt, const int32_t* kv_indices,
                                const int64_t* kv_start, const int32_t* kv_len, const int32_t* qo_indptr, const int32_t* tok_seq,
                                float scale, float cap, void* out, int64_t n_tok, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                                int n_split, float* part, int64_t window, const float* r1, const float* r2, const double* vfreq,
                                int v_interleaved, const void* gate, int64_t gate_stride, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_softcap_attn: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_tok <= 65535 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 4096 && vdim > 0 && vdim <= 512,
                NVX_EINVAL, "nvx_softcap_attn: bad sizes (at most 65535 tokens a step, key size <= 4096, value size <= 512)");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(q && k_cache && v_cache && kv_indices && kv_start && kv_len && out, NVX_EINVAL, "nvx_softcap_attn: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_softcap_attn: tok_seq and qo_indptr go together");
    NVX_REQUIRE((r1 != nullptr) == (r2 != nullptr), NVX_EINVAL, "nvx_softcap_attn: the distance penalty takes both of its numbers per head");
    NVX_REQUIRE(window >= 0 && window < (1ll << 31), NVX_EINVAL, "nvx_softcap_attn: bad window");
    NVX_REQUIRE(!vfreq || vdim % 2 == 0, NVX_EINVAL, "nvx_softcap_attn: a read-out that is turned back has an even size");
    NVX_REQUIRE(!gate || gate_stride >= heads * vdim, NVX_EINVAL, "nvx_softcap_attn: row stride of the gate");
    const size_t lds = (size_t)(dim + 4 * vdim + 8) * sizeof(float);
    NVX_REQUIRE(n_split >= 1 && n_split <= 64 && (n_split == 1 || part), NVX_EINVAL, "nvx_softcap_attn: a key split needs its workspace");
    const dim3 grid((unsigned)heads, (unsigned)n_tok, (unsigned)n_split);
#define NVX_CAP_ATTN_V(EPL, VEC)                                                                                                          \
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL((softcap_attn_kernel<A_, EPL, VEC && sizeof(A_) == 2>), grid, dim3(256), lds, (hipStream_t)stream,     \
                                         (const A_*)q, (const A_*)k_cache, (const A_*)v_cache, kv_indices, kv_start, kv_len, qo_indptr,      \
                                         tok_seq, scale, cap, (A_*)out, (int)heads, (int)kv_heads, (int)dim, (int)vdim,       \
                                         (int)nvx_aligned16(v_cache), n_split, part, (int)window, r1, r2, vfreq, v_interleaved, \
                                         (const A_*)gate, gate_stride))
#define NVX_CAP_ATTN(EPL) do { if (vec) NVX_CAP_ATTN_V(EPL, true); else NVX_CAP_ATTN_V(EPL, false); } while (0)
    const bool vec = fmt != 2 && dim % 8 == 0 && nvx_aligned16(k_cache);
    if (vdim <= 64) NVX_CAP_ATTN(1);
    else if (vdim <= 128) NVX_CAP_ATTN(2);
    else if (vdim <= 256) NVX_CAP_ATTN(4);
    else NVX_CAP_ATTN(8);
#undef NVX_CAP_ATTN_V
    if (n_split > 1)
        NVX_FMT_CALL(fmt, hipLaunchKernelGGL(softcap_merge_kernel<A_>, dim3((unsigned)(n_tok * heads)), dim3(64), 0, (hipStream_t)stream,
                                             (const float*)part, n_split, (A_*)out, (int)vdim, (int)heads, kv_len, qo_indptr, tok_seq, vfreq,
                                             v_interleaved, (const A_*)gate, gate_stride));
#undef NVX_CAP_ATTN
    return nvx_check_launch("nvx_softcap_attn");
}
