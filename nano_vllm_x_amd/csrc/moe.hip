// Mixture of small gated feed-forward experts; a choice's weight scales the chosen expert's INPUT (sigmoid routers) or its
// OUTPUT (weight_out: fixed weights from a table).
//   - nvx_moe_route: the `top` largest router logits of every token -> expert ids and sigmoid scores (float32);
//   - nvx_moe_route_softmax: softmax scores, experts in groups of which only the best may be chosen, weights renormalised;
//   - nvx_moe_expert_rows: a token's experts evaluated row by row of their weights: the form for steps of few tokens, where
//     every chosen expert's weights have to be streamed once per token anyway;
//   - nvx_moe_order / nvx_moe_scatter_rows / nvx_moe_glu / nvx_moe_gather_rows: the pieces around per-expert matrix products
//     for steps of many tokens (the expert order of the (token, choice) pairs and the experts' counts, scaled inputs gathered
//     into that order, the gated activation, the tokens' results summed back).
// Expert:  g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit), y = g sigmoid(alpha g) (u + shift), out = W_down y
// (limit = infinity, alpha = 1, shift = 0: silu(g) u).
#include "fmt_dev.h"

namespace NVX_NS {

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int n_exp, int top, int32_t* __restrict__ idx,
                                                       float* __restrict__ wts, int64_t n_tok) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_tok) return;
    const float* z = logits + t * n_exp;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bz = -INFINITY;
        for (int e = 0; e < n_exp; ++e) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= idx[t * top + j] == e;
            if (!taken && (best < 0 || z[e] > bz)) { best = e; bz = z[e]; }
        }
        idx[t * top + k] = best;
        wts[t * top + k] = sigmoid_f(bz);
    }
}

// Softmax router with groups: scores = softmax(logits) over all experts; the experts form n_groups equal groups of neighbours, a
// group counts as its best score, and only experts of the keep_groups best groups can be chosen (n_groups <= 1: all of them);
// the `top` largest scores among those are chosen (ties: the lower id) and their scores, divided by their sum + norm_eps, are the
// weights.  One thread per token; everything float32.
__global__ __launch_bounds__(256) void moe_route_softmax_kernel(const float* __restrict__ logits, int n_exp, int top, int n_groups,
                                                               int keep_groups, float norm_eps, int32_t* __restrict__ idx,
                                                               float* __restrict__ wts, int64_t n_tok) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_tok) return;
    const float* z = logits + t * n_exp;
    float zmax = -INFINITY;
    for (int e = 0; e < n_exp; ++e) zmax = fmaxf(zmax, z[e]);
    float denom = 0.f;
    for (int e = 0; e < n_exp; ++e) denom += expf(z[e] - zmax);
    // the groups that stay: keep_groups times the best group not yet taken (a group's score is its largest logit: the softmax keeps the order)
    uint64_t kept[4] = {0, 0, 0, 0};                       // n_groups <= 256
    const bool grouped = n_groups > 1 && keep_groups < n_groups;
    const int per = grouped ? n_exp / n_groups : n_exp;
    if (grouped) {
        for (int k = 0; k < keep_groups; ++k) {
            int best = -1;
            float bz = -INFINITY;
            for (int g = 0; g < n_groups; ++g) {
                if ((kept[g >> 6] >> (g & 63)) & 1) continue;
                float gm = -INFINITY;
                for (int e = g * per; e < (g + 1) * per; ++e) gm = fmaxf(gm, z[e]);
                if (best < 0 || gm > bz) { best = g; bz = gm; }
            }
            kept[best >> 6] |= 1ull << (best & 63);
        }
    }
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bz = -INFINITY;
        for (int e = 0; e < n_exp; ++e) {
            if (grouped) { const int g = e / per; if (!((kept[g >> 6] >> (g & 63)) & 1)) continue; }
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= idx[t * top + j] == e;
            if (!taken && (best < 0 || z[e] > bz)) { best = e; bz = z[e]; }
        }
        idx[t * top + k] = best;
        const float sc = expf(bz - zmax) / denom;
        wts[t * top + k] = sc;
        sum += sc;
    }
    for (int k = 0; k < top; ++k) wts[t * top + k] /= (sum + norm_eps);
}

__device__ __forceinline__ float glu_act(float g, float u, float limit, float alpha, float shift) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoid_f(alpha * g) * (u + shift);
}

// A token's experts row by row.  w_gu: (experts, 2 * ff, width) rows [gate | up]; w_d: (experts, width, ff).  Two launches, both
// with a workgroup per 32 weight rows so that a step of a few tokens still fills the chip: the hidden activations of every
// (token, choice) pair into a float32 workspace, then the output rows summed over a token's choices.  A wave takes 8 rows; its
// lanes walk a row 8 elements at a time (16-byte loads) where the format is 16-bit and the rows are 16-byte aligned.
template <typename A, bool VEC>
__device__ __forceinline__ float lane_dot(const A* __restrict__ wrow, const float* __restrict__ xs, int n, int lane) {
    float acc = 0.f;
    if constexpr (VEC) {
        typedef A vec8 __attribute__((ext_vector_type(8)));
        for (int c = lane * 8; c < n; c += 512) {
            const vec8 v = *reinterpret_cast<const vec8*>(wrow + c);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc += (float)v[i] * xs[c + i];
        }
    } else {
        for (int c = lane; c < n; c += 64) acc += ld_f(wrow, c) * xs[c];
    }
    return acc;
}

// Two rows against one LDS vector, with the loads of four 512-element steps of both rows (eight 16-byte loads a lane) issued
// before the first product: a wave alone then keeps 8 KB in flight instead of waiting out one load's latency per step.
template <typename A, bool VEC>
__device__ __forceinline__ void lane_dot2(const A* __restrict__ ra, const A* __restrict__ rb, const float* __restrict__ xs, int n, int lane,
                                          float& out_a, float& out_b) {
    float a = 0.f, b = 0.f;
    if constexpr (VEC) {
        typedef A vec8 __attribute__((ext_vector_type(8)));
        int c = lane * 8;
        for (; c + 1536 < n; c += 2048) {
            vec8 va[4], vb[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                va[s] = *reinterpret_cast<const vec8*>(ra + c + 512 * s);
                vb[s] = *reinterpret_cast<const vec8*>(rb + c + 512 * s);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float x = xs[c + 512 * s + i];
                    a += (float)va[s][i] * x;
                    b += (float)vb[s][i] * x;
                }
            }
        }
        for (; c < n; c += 512) {
            const vec8 va = *reinterpret_cast<const vec8*>(ra + c);
            const vec8 vb = *reinterpret_cast<const vec8*>(rb + c);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = xs[c + i];
                a += (float)va[i] * x;
                b += (float)vb[i] * x;
            }
        }
    } else {
        for (int c = lane; c < n; c += 64) {
            const float x = xs[c];
            a += ld_f(ra, c) * x;
            b += ld_f(rb, c) * x;
        }
    }
    out_a = a;
    out_b = b;
}

constexpr int MOE_ROWS = 32;      // weight rows per workgroup (8 per wave)

template <typename A, bool VEC>
__global__ __launch_bounds__(256) void moe_rows_up_kernel(const A* __restrict__ h, int64_t h_stride, const int32_t* __restrict__ idx,
                                                         const float* __restrict__ wts, int top, const A* __restrict__ w_gu, float limit,
                                                         float alpha, float shift, int weight_out, float* __restrict__ y, int width, int ff) {
    extern __shared__ float sm[];      // the scaled input (width)
    const int64_t t = blockIdx.z;
    const int k = blockIdx.y;
    const int e = idx[t * top + k];
    const float wt = weight_out ? 1.0f : wts[t * top + k];
    for (int c = threadIdx.x; c < width; c += 256) sm[c] = (float)(A)(wt * ld_f(h, t * h_stride + c));
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const A* wg = w_gu + (int64_t)e * 2 * ff * width;
    float g[MOE_ROWS / 4], u[MOE_ROWS / 4];
#pragma unroll
    for (int i = 0; i < MOE_ROWS / 4; ++i) {         // all rows' loads in flight before the first reduction
        const int j = blockIdx.x * MOE_ROWS + wave * (MOE_ROWS / 4) + i;
        const int jc = j < ff ? j : ff - 1;
        lane_dot2<A, VEC>(wg + (int64_t)jc * width, wg + (int64_t)(ff + jc) * width, sm, width, lane, g[i], u[i]);
    }
#pragma unroll
    for (int i = 0; i < MOE_ROWS / 4; ++i) {
        const int j = blockIdx.x * MOE_ROWS + wave * (MOE_ROWS / 4) + i;
        const float gs = wave_sum(g[i]), us = wave_sum(u[i]);
        if (lane == 0 && j < ff) y[(t * top + k) * ff + j] = (float)(A)glu_act((float)(A)gs, (float)(A)us, limit, alpha, shift);
    }
}

template <typename A, bool VEC>
__global__ __launch_bounds__(256) void moe_rows_down_kernel(const float* __restrict__ y, const int32_t* __restrict__ idx,
                                                           const float* __restrict__ wts, int top, int weight_out,
                                                           const A* __restrict__ w_d, A* __restrict__ out, int width, int ff) {
    extern __shared__ float sm[];      // one choice's hidden activations (ff)
    const int64_t t = blockIdx.y;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float o[MOE_ROWS / 4];
#pragma unroll
    for (int i = 0; i < MOE_ROWS / 4; ++i) o[i] = 0.f;
    for (int k = 0; k < top; ++k) {
        __syncthreads();
        for (int j = threadIdx.x; j < ff; j += 256) sm[j] = y[(t * top + k) * ff + j];
        __syncthreads();
        const A* wd = w_d + (int64_t)idx[t * top + k] * width * ff;
        float part[MOE_ROWS / 4];
#pragma unroll
        for (int i = 0; i < MOE_ROWS / 4; i += 2) {
            const int c = blockIdx.x * MOE_ROWS + wave * (MOE_ROWS / 4) + i;
            lane_dot2<A, VEC>(wd + (int64_t)(c < width ? c : width - 1) * ff, wd + (int64_t)(c + 1 < width ? c + 1 : width - 1) * ff, sm, ff, lane,
                              part[i], part[i + 1]);
        }
        const float wo = weight_out ? wts[t * top + k] : 1.0f;
#pragma unroll
        for (int i = 0; i < MOE_ROWS / 4; ++i) o[i] += wo * (float)(A)wave_sum(part[i]);
    }
#pragma unroll
    for (int i = 0; i < MOE_ROWS / 4; ++i) {
        const int c = blockIdx.x * MOE_ROWS + wave * (MOE_ROWS / 4) + i;
        if (c < width && lane == 0) st_f(out, t * (int64_t)width + c, o[i]);
    }
}

// xs[dst[r]] = wts[r] * h[r / top]  for every (token, choice) pair r: the experts' inputs in expert order
template <typename A>
__global__ __launch_bounds__(256) void moe_scatter_rows_kernel(const A* __restrict__ h, int64_t h_stride, const float* __restrict__ wts,
                                                              const int64_t* __restrict__ dst, int top, A* __restrict__ xs, int width) {
    const int64_t r = blockIdx.x;
    const int64_t t = r / top;
    const float wt = wts ? wts[r] : 1.0f;
    A* o = xs + dst[r] * (int64_t)width;
    for (int c = threadIdx.x; c < width; c += 256) st_f(o, c, wt * ld_f(h, t * h_stride + c));
}

// y[r][j] = act(gu[r][j], gu[r][ff + j])
template <typename A>
__global__ __launch_bounds__(256) void moe_glu_kernel(const A* __restrict__ gu, A* __restrict__ y, float limit, float alpha, float shift,
                                                     int64_t rows, int ff) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < rows * ff; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / ff;
        const int j = (int)(i % ff);
        st_f(y, i, glu_act(ld_f(gu, r * 2 * ff + j), ld_f(gu, r * 2 * ff + ff + j), limit, alpha, shift));
    }
}

// The same for 16-bit formats, eight neighbouring entries of a row per thread as one 16-byte load of each half and one store
// (ff8 = ff / 8; rows start on 16-byte borders).
template <typename A>
__global__ __launch_bounds__(256) void moe_glu_vec8_kernel(const A* __restrict__ gu, A* __restrict__ y, float limit, float alpha, float shift,
                                                          int64_t rows, int ff8) {
    union Pack { uint4 v; A a[8]; };
    const int64_t n = rows * ff8;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / ff8;
        const int64_t j = (i - r * ff8) * 8;
        const A* row = gu + r * 16 * ff8;
        Pack g, u, o;
        g.v = *reinterpret_cast<const uint4*>(row + j);
        u.v = *reinterpret_cast<const uint4*>(row + (int64_t)ff8 * 8 + j);
#pragma unroll
        for (int k = 0; k < 8; ++k) o.a[k] = (A)glu_act((float)g.a[k], (float)u.a[k], limit, alpha, shift);
        *reinterpret_cast<uint4*>(y + i * 8) = o.v;
    }
}

// out[t] = sum_k wts[t * top + k] * ys[dst[t * top + k]]   (wts == null: ones)
template <typename A>
__global__ __launch_bounds__(256) void moe_gather_rows_kernel(const A* __restrict__ ys, const int64_t* __restrict__ dst,
                                                             const float* __restrict__ wts, int top, A* __restrict__ out, int width) {
    const int64_t t = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += 256) {
        float o = 0.f;
        for (int k = 0; k < top; ++k) o += (wts ? wts[t * top + k] : 1.0f) * ld_f(ys, dst[t * top + k] * (int64_t)width + c);
        st_f(out, t * (int64_t)width + c, o);
    }
}


// Expert order of the (token, choice) pairs: dst[r] = position of pair r when the pairs are sorted by expert, pairs of one
// expert keeping their order; counts[e] = pairs of expert e.  One workgroup: a thread takes a contiguous run of pairs, counts
// them per expert into LDS (cnt[e][thread]), the prefix sums over (expert, thread) give every thread its first position per
// expert, and a second walk over the same run hands the positions out.  n_exp * 256 counters must fit LDS.
__global__ __launch_bounds__(256) void moe_order_kernel(const int32_t* __restrict__ idx, int64_t n, int n_exp, int64_t* __restrict__ dst,
                                                       int32_t* __restrict__ counts) {
    extern __shared__ int cnt[];      // n_exp rows of 256, then n_exp bases
    int* base = cnt + n_exp * 256;
    const int tid = threadIdx.x;
    const int64_t per = (n + 255) / 256, lo = tid * per, hi = lo + per < n ? lo + per : n;
    for (int e = 0; e < n_exp; ++e) cnt[e * 256 + tid] = 0;
    for (int64_t r = lo; r < hi; ++r) {
        const int e = idx[r];
        if (e >= 0 && e < n_exp) cnt[e * 256 + tid] += 1;
    }
    __syncthreads();
    for (int e = tid; e < n_exp; e += 256) {       // a thread per expert: exclusive prefix over the threads' counts
        int run = 0;
        for (int j = 0; j < 256; ++j) { const int c = cnt[e * 256 + j]; cnt[e * 256 + j] = run; run += c; }
        base[e] = run;
        counts[e] = run;
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < n_exp; ++e) { const int c = base[e]; base[e] = run; run += c; }
    }
    __syncthreads();
    for (int64_t r = lo; r < hi; ++r) {
        const int e = idx[r];
        if (e >= 0 && e < n_exp) dst[r] = base[e] + cnt[e * 256 + tid]++;
    }
}

}  // namespace NVX_NS

using namespace NVX_NS;

extern "C" int64_t nvx_moe_order_max_experts(void) { return (64 * 1024 / 4) / 257; }

extern "C" int nvx_moe_order(const int32_t* idx, int64_t n, int64_t n_exp, int64_t* dst, int32_t* counts, nvx_stream_t stream) {
    NVX_REQUIRE(n >= 0 && n < (1ll << 31) && n_exp > 0 && n_exp <= nvx_moe_order_max_experts(), NVX_EINVAL,
                "nvx_moe_order: bad sizes (the experts' counters must fit LDS)");
    NVX_REQUIRE(idx && dst && counts, NVX_EINVAL, "nvx_moe_order: null pointer");
    hipLaunchKernelGGL(moe_order_kernel, dim3(1), dim3(256), (size_t)(n_exp * 257) * sizeof(int), (hipStream_t)stream, idx, n, (int)n_exp, dst,
                       counts);
    return nvx_check_launch("nvx_moe_order");
}

extern "C" int nvx_moe_route(const float* logits, int64_t n_tok, int64_t n_exp, int64_t top, int32_t* idx, float* wts, nvx_stream_t stream) {
    NVX_REQUIRE(n_tok >= 0 && n_exp > 0 && n_exp < (1 << 20) && top > 0 && top <= n_exp, NVX_EINVAL, "nvx_moe_route: bad sizes");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(logits && idx && wts, NVX_EINVAL, "nvx_moe_route: null pointer");
    hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)((n_tok + 255) / 256)), dim3(256), 0, (hipStream_t)stream, logits, (int)n_exp, (int)top,
                       idx, wts, n_tok);
    return nvx_check_launch("nvx_moe_route");
}

extern "C" int nvx_moe_route_softmax(const float* logits, int64_t n_tok, int64_t n_exp, int64_t top, int64_t n_groups, int64_t keep_groups,
                                     float norm_eps, int32_t* idx, float* wts, nvx_stream_t stream) {
    NVX_REQUIRE(n_tok >= 0 && n_exp > 0 && n_exp < (1 << 20) && top > 0 && top <= n_exp, NVX_EINVAL, "nvx_moe_route_softmax: bad sizes");
    NVX_REQUIRE(n_groups >= 0 && n_groups <= 256 && (n_groups <= 1 || (n_exp % n_groups == 0 && keep_groups >= 1 && keep_groups <= n_groups &&
                                                                      keep_groups * (n_exp / n_groups) >= top)),
                NVX_EINVAL, "nvx_moe_route_softmax: groups must divide the experts (at most 256 groups) and the kept groups must hold `top` experts");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(logits && idx && wts, NVX_EINVAL, "nvx_moe_route_softmax: null pointer");
    hipLaunchKernelGGL(moe_route_softmax_kernel, dim3((unsigned)((n_tok + 255) / 256)), dim3(256), 0, (hipStream_t)stream, logits, (int)n_exp,
                       (int)top, (int)n_groups, (int)keep_groups, norm_eps, idx, wts, n_tok);
    return nvx_check_launch("nvx_moe_route_softmax");
}

extern "C" int64_t nvx_moe_expert_rows_max_width(int64_t ff) {
    return ff > 0 && ff <= 12288 ? 12288 : 0;      // a row of either size waits in LDS as float32
}

template <typename A>
static void launch_moe_rows(const void* h, int64_t h_stride, const int32_t* idx, const float* wts, int top, const void* w_gu, const void* w_d,
                            float limit, float alpha, float shift, int weight_out, float* ws, void* out, int64_t n_tok, int width, int ff,
                            hipStream_t s) {
    const bool vec = sizeof(A) == 2 && width % 8 == 0 && ff % 8 == 0 && nvx_aligned16(w_gu) && nvx_aligned16(w_d);
    const dim3 up((unsigned)((ff + MOE_ROWS - 1) / MOE_ROWS), (unsigned)top, (unsigned)n_tok);
    const dim3 down((unsigned)((width + MOE_ROWS - 1) / MOE_ROWS), (unsigned)n_tok);
    if (vec) {
        hipLaunchKernelGGL((moe_rows_up_kernel<A, true>), up, dim3(256), (size_t)width * sizeof(float), s, (const A*)h, h_stride, idx, wts, top,
                           (const A*)w_gu, limit, alpha, shift, weight_out, ws, width, ff);
        hipLaunchKernelGGL((moe_rows_down_kernel<A, true>), down, dim3(256), (size_t)ff * sizeof(float), s, (const float*)ws, idx, wts, top,
                           weight_out, (const A*)w_d, (A*)out, width, ff);
    } else {
        hipLaunchKernelGGL((moe_rows_up_kernel<A, false>), up, dim3(256), (size_t)width * sizeof(float), s, (const A*)h, h_stride, idx, wts, top,
                           (const A*)w_gu, limit, alpha, shift, weight_out, ws, width, ff);
        hipLaunchKernelGGL((moe_rows_down_kernel<A, false>), down, dim3(256), (size_t)ff * sizeof(float), s, (const float*)ws, idx, wts, top,
                           weight_out, (const A*)w_d, (A*)out, width, ff);
    }
}

extern "C" int nvx_moe_expert_rows(const void* h, int64_t h_stride, int fmt, const int32_t* idx, const float* wts, int64_t top,
                                   const void* w_gu, const void* w_d, int64_t n_exp, float limit, float alpha, float shift, int weight_out,
                                   float* ws, void* out, int64_t n_tok, int64_t width, int64_t ff, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_moe_expert_rows: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_tok <= 65535 && top > 0 && top <= 65535 && n_exp > 0 && width > 0 && ff > 0 && h_stride >= width, NVX_EINVAL,
                "nvx_moe_expert_rows: bad sizes (at most 65535 tokens a step)");
    NVX_REQUIRE(width <= nvx_moe_expert_rows_max_width(ff), NVX_EUNSUPPORTED, "nvx_moe_expert_rows: a row or the hidden size does not fit LDS");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(h && idx && wts && w_gu && w_d && ws && out, NVX_EINVAL, "nvx_moe_expert_rows: null pointer");
    NVX_FMT_CALL(fmt, launch_moe_rows<A_>(h, h_stride, idx, wts, (int)top, w_gu, w_d, limit, alpha, shift, weight_out, ws, out, n_tok, (int)width, (int)ff,
                                          (hipStream_t)stream));
    return nvx_check_launch("nvx_moe_expert_rows");
}

extern "C" int nvx_moe_scatter_rows(const void* h, int64_t h_stride, int fmt, const float* wts, const int64_t* dst, int64_t top, void* xs,
                                    int64_t n_tok, int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && n_tok >= 0 && top > 0 && width > 0 && h_stride >= width && n_tok * top < (1ll << 31), NVX_EINVAL,
                "nvx_moe_scatter_rows: bad arguments");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(h && dst && xs, NVX_EINVAL, "nvx_moe_scatter_rows: null pointer");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(moe_scatter_rows_kernel<A_>, dim3((unsigned)(n_tok * top)), dim3(256), 0, (hipStream_t)stream,
                                         (const A_*)h, h_stride, wts, dst, (int)top, (A_*)xs, (int)width));
    return nvx_check_launch("nvx_moe_scatter_rows");
}

extern "C" int nvx_moe_glu(const void* gu, int fmt, float limit, float alpha, float shift, void* y, int64_t rows, int64_t ff,
                           nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && rows >= 0 && ff > 0, NVX_EINVAL, "nvx_moe_glu: bad arguments");
    if (rows == 0) return NVX_OK;
    NVX_REQUIRE(gu && y, NVX_EINVAL, "nvx_moe_glu: null pointer");
    if (fmt != 2 && ff % 8 == 0 && nvx_aligned16(gu) && nvx_aligned16(y)) {
        int64_t blocks = (rows * (ff / 8) + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        if (fmt == 0)
            hipLaunchKernelGGL(moe_glu_vec8_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const __bf16*)gu, (__bf16*)y,
                               limit, alpha, shift, rows, (int)(ff / 8));
        else
            hipLaunchKernelGGL(moe_glu_vec8_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const _Float16*)gu,
                               (_Float16*)y, limit, alpha, shift, rows, (int)(ff / 8));
        return nvx_check_launch("nvx_moe_glu");
    }
    int64_t blocks = (rows * ff + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(moe_glu_kernel<A_>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const A_*)gu, (A_*)y, limit,
                                         alpha, shift, rows, (int)ff));
    return nvx_check_launch("nvx_moe_glu");
}

extern "C" int nvx_moe_gather_rows(const void* ys, int fmt, const int64_t* dst, const float* wts, int64_t top, void* out, int64_t n_tok,
                                   int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && n_tok >= 0 && n_tok < (1ll << 31) && top > 0 && width > 0, NVX_EINVAL, "nvx_moe_gather_rows: bad arguments");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(ys && dst && out, NVX_EINVAL, "nvx_moe_gather_rows: null pointer");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(moe_gather_rows_kernel<A_>, dim3((unsigned)n_tok), dim3(256), 0, (hipStream_t)stream, (const A_*)ys, dst,
                                         wts, (int)top, (A_*)out, (int)width));
    return nvx_check_launch("nvx_moe_gather_rows");
}
