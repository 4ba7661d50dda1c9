// Sublayer boundaries of stacks whose residual stream is float32, whose norms work on groups of a row, and whose sublayer
// results pass a learned sigmoid gate before they are added:
//   - gated residual + grouped RMS norm, one launch per boundary (optionally the result is first formed as the mean of two
//     RMS-normed branch outputs);
//   - per-head RMS norm of a recurrence's or attention's read-out, times a weight, times an output gate;
//   - stacks that norm a sublayer's OUTPUT instead of its input: the (weighted sum of one or two) results divided by its root
//     mean square, times a weight (one number or one per channel), added to the stream, which the next sublayer reads as it is;
//   - the two ends of such a stack: scaled embedding rows into the stream, and logits through cap * tanh(. / cap).
// Norms, gates and the stream are float32 in every activation format.
#include "fmt_dev.h"

namespace NVX_NS {

// Per token t (one workgroup):
//   r = y[t]                                                   (y2 == null)
//   r = (y[t] / rms(y[t]) * w_y + y2[t] / rms(y2[t]) * w_y2) / 2     (y2 != null; rms over the whole row)
//   r *= sigmoid(gate[t] + gate_bias)                          (gate != null)
//   x[t] += mult * r                                           (y != null)
//   h[t] = x[t], each of `groups` consecutive slices divided by its own root mean square, times w_norm   (w_norm != null)
template <typename A>
__global__ __launch_bounds__(256) void gated_residual_norm_kernel(
    const A* __restrict__ y, int64_t y_stride, const A* __restrict__ y2, int64_t y2_stride, const float* __restrict__ w_y,
    const float* __restrict__ w_y2, const A* __restrict__ gate, int64_t gate_stride, const float* __restrict__ gate_bias, float mult,
    float* __restrict__ x, const float* __restrict__ w_norm, int groups, float eps, A* __restrict__ h_out, int width) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const int64_t row = t * (int64_t)width;
    const A* yr = y ? y + t * y_stride : nullptr;
    const A* y2r = y2 ? y2 + t * y2_stride : nullptr;
    const A* gr = gate ? gate + t * gate_stride : nullptr;
    float r1 = 1.f, r2 = 1.f;
    if (y2r) {
        float a = 0.f, b = 0.f;
        for (int c = threadIdx.x; c < width; c += 256) {
            const float u = ld_f(yr, c), v = ld_f(y2r, c);
            a += u * u;
            b += v * v;
        }
        r1 = 1.0f / sqrtf(block256_sum(a, red) / (float)width + eps);
        r2 = 1.0f / sqrtf(block256_sum(b, red) / (float)width + eps);
    }
    const int gs = width / groups;
    for (int g = 0; g < groups; ++g) {
        const int lo = g * gs, hi = lo + gs;
        float ss = 0.f;
        for (int c = lo + threadIdx.x; c < hi; c += 256) {
            float xv = x[row + c];
            if (yr) {
                float r = ld_f(yr, c);
                if (y2r) r = 0.5f * (r * r1 * w_y[c] + ld_f(y2r, c) * r2 * w_y2[c]);
                if (gr) r *= sigmoid_f(ld_f(gr, c) + (gate_bias ? gate_bias[c] : 0.f));
                xv += mult * r;
                x[row + c] = xv;
            }
            ss += xv * xv;
        }
        if (!w_norm) continue;
        const float rn = 1.0f / sqrtf(block256_sum(ss, red) / (float)gs + eps);
        for (int c = lo + threadIdx.x; c < hi; c += 256) st_f(h_out, row + c, x[row + c] * rn * w_norm[c]);   // own stores, read back
    }
}

// Per token t (one workgroup):
//   r = a * y[t] (+ b * y2[t]);  x[t] += r / rms(r) * w_post                  (y != null; w_post: one number or `width` of them)
//   h[t] = x[t] / rms(x[t]) * w_next  (w_next != null)   or   h[t] = x[t]     (h_out != null)
template <typename A>
__global__ __launch_bounds__(256) void postnorm_residual_kernel(const A* __restrict__ y, int64_t y_stride, const A* __restrict__ y2,
                                                               int64_t y2_stride, float a, float b, const float* __restrict__ w_post,
                                                               int w_post_n, float* __restrict__ x, const float* __restrict__ w_next,
                                                               int w_next_n, float eps, A* __restrict__ h_out, int width) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    float* xr = x + t * (int64_t)width;
    const A* yr = y ? y + t * y_stride : nullptr;
    const A* y2r = y2 ? y2 + t * y2_stride : nullptr;
    float rn = 0.f;
    if (yr) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < width; c += 256) {
            const float r = a * ld_f(yr, c) + (y2r ? b * ld_f(y2r, c) : 0.f);
            ss += r * r;
        }
        rn = 1.0f / sqrtf(block256_sum(ss, red) / (float)width + eps);
    }
    float sx = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
        float xv = xr[c];
        if (yr) {
            const float r = a * ld_f(yr, c) + (y2r ? b * ld_f(y2r, c) : 0.f);
            xv += r * rn * w_post[w_post_n == 1 ? 0 : c];
            xr[c] = xv;
        }
        sx += xv * xv;
    }
    if (!h_out) return;
    A* hr = h_out + t * (int64_t)width;
    if (w_next) {
        const float rx = 1.0f / sqrtf(block256_sum(sx, red) / (float)width + eps);
        for (int c = threadIdx.x; c < width; c += 256) st_f(hr, c, xr[c] * rx * w_next[w_next_n == 1 ? 0 : c]);     // own stores, read back
    } else {
        for (int c = threadIdx.x; c < width; c += 256) st_f(hr, c, xr[c]);
    }
}

// Several residual streams per token (x: (tokens, streams, width) float32) and the sublayer boundary between them.  Per token t:
//   with a result y:   r = y[t] * scale (scale: one number per channel, or none);
//                      every stream at once from the old ones:  x_j' = sum_s mix[s][j] x_s + w_out[j] r      (mix indexed [from][to])
//   without one:       x_j' = x_j  (x_in may be ONE row per token that all streams start from: in_stream_stride 0)
//   then what the next sublayer reads:  u = sum_j w_in[j] x_j'  (w_in null: the plain sum),  h[t] = u / rms(u) * w_norm.
// A thread holds the old values of its columns for all streams before it writes any, so x_in may be x_out.  u waits in LDS for
// the row's mean square.
template <typename A, int MAXS>
__global__ __launch_bounds__(256) void hyper_mix_kernel(const float* x_in, int64_t in_tok_stride, int64_t in_stream_stride,
                                                       const A* __restrict__ y, int64_t y_stride, const float* __restrict__ scale,
                                                       const float* __restrict__ mix, const float* __restrict__ w_out,
                                                       const float* __restrict__ w_in, const float* __restrict__ w_norm, float eps,
                                                       float* x_out, A* __restrict__ h_out, int n_streams, int width) {
    extern __shared__ float su[];                 // width
    __shared__ float s_mix[MAXS * MAXS], s_out[MAXS], s_in[MAXS], red[4];
    const int64_t t = blockIdx.x;
    for (int i = threadIdx.x; i < n_streams * n_streams; i += 256) s_mix[(i / n_streams) * MAXS + (i % n_streams)] = mix ? mix[i] : 0.f;
    for (int i = threadIdx.x; i < n_streams; i += 256) { s_out[i] = w_out ? w_out[i] : 0.f; s_in[i] = w_in ? w_in[i] : 1.0f; }
    __syncthreads();
    const float* xr = x_in + t * in_tok_stride;
    float* xo = x_out + t * (int64_t)n_streams * width;
    const A* yr = y ? y + t * y_stride : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
        float old[MAXS];
#pragma unroll
        for (int s = 0; s < MAXS; ++s) old[s] = s < n_streams ? xr[s * in_stream_stride + c] : 0.f;
        const float r = yr ? ld_f(yr, c) * (scale ? scale[c] : 1.0f) : 0.f;
        float u = 0.f;
#pragma unroll
        for (int j = 0; j < MAXS; ++j) {
            if (j < n_streams) {
                float v = old[j];
                if (yr) {
                    v = s_out[j] * r;
#pragma unroll
                    for (int s = 0; s < MAXS; ++s) if (s < n_streams) v += s_mix[s * MAXS + j] * old[s];
                }
                if (yr || x_out != x_in || in_stream_stride == 0) xo[(int64_t)j * width + c] = v;
                u += s_in[j] * v;
            }
        }
        su[c] = u;
        ss += u * u;
    }
    if (!h_out) return;
    const float rn = 1.0f / sqrtf(block256_sum(ss, red) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += 256) st_f(h_out, t * (int64_t)width + c, su[c] * rn * (w_norm ? w_norm[c] : 1.0f));
}

// x[t] = table[ids[t]] * scale (float32), h[t] = the same in the activations' format
template <typename A>
__global__ __launch_bounds__(256) void embed_scale_kernel(const int64_t* __restrict__ ids, const A* __restrict__ table, int64_t vocab, float scale,
                                                         float* __restrict__ x, A* __restrict__ h, int width) {
    const int64_t t = blockIdx.x;
    int64_t id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int c = threadIdx.x; c < width; c += 256) {
        const float v = ld_f(table, id * width + c) * scale;
        x[t * (int64_t)width + c] = v;
        if (h) st_f(h, t * (int64_t)width + c, v);
    }
}

template <typename A>
__global__ __launch_bounds__(256) void tanh_cap_kernel(const A* __restrict__ in, float cap, float* __restrict__ out, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const float z = ld_f(in, i);
        out[i] = cap > 0.f ? cap * tanhf(z / cap) : z;
    }
}

// One wave per (token, head): out = o / rms(o) * w * gate, with gate = 1 (kind 0), sigmoid(z) (1) or z * sigmoid(z) (2) of
// the gate pre-activations z (same layout as the output).  w has heads * vdim entries, or vdim shared by the heads.
template <typename A>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, int w_shared,
                                                            const A* __restrict__ gate, int64_t gate_stride, int kind, float eps,
                                                            A* __restrict__ out, int64_t n_rows, int heads, int vdim) {
    const int64_t idx = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (idx >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = idx / heads;
    const int hd = (int)(idx % heads);
    const int64_t base = t * (int64_t)heads * vdim + (int64_t)hd * vdim;
    float ss = 0.f;
    for (int e = lane; e < vdim; e += 64) { const float v = o[base + e]; ss += v * v; }
    const float rn = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
    for (int e = lane; e < vdim; e += 64) {
        float v = o[base + e] * rn * w[w_shared ? e : hd * vdim + e];
        if (kind) {
            const float z = ld_f(gate, t * gate_stride + (int64_t)hd * vdim + e);
            v *= kind == 1 ? sigmoid_f(z) : z * sigmoid_f(z);
        }
        st_f(out, base + e, v);
    }
}


// Projections onto FEW outputs or from FEW inputs, in float32: gate and router logits (outputs = heads or experts), the two
// halves of a low-rank decay.  out[t][n] = sum_k W[n][k] * f(x[t][k]), f = identity or tanh; W float32 (n_out, k_in).  A
// workgroup takes TOK tokens: their inputs wait in LDS as float32, every weight is read once for the TOK of them.  Wide
// inputs: a wave per output, lanes over k.  Narrow inputs (k_in < 256): a thread per output.  No workspace, no atomics: the
// sums have one order, and the launch can be captured.
template <typename A, int TOK>
__global__ __launch_bounds__(256) void skinny_proj_kernel(const A* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                         int in_act, float* __restrict__ out, int64_t n_tok, int n_out, int k_in,
                                                         int out_per_block) {
    extern __shared__ float xs[];      // TOK rows of k_in
    const int64_t t0 = (int64_t)blockIdx.x * TOK;
    const int nt = (int)(n_tok - t0 < TOK ? n_tok - t0 : TOK);
    for (int i = threadIdx.x; i < TOK * k_in; i += 256) {
        const int tt = i / k_in, k = i % k_in;
        float v = tt < nt ? ld_f(x, (t0 + tt) * x_stride + k) : 0.f;
        xs[i] = in_act == 1 ? tanhf(v) : v;
    }
    __syncthreads();
    const int n_lo = blockIdx.y * out_per_block;
    const int n_hi = n_lo + out_per_block < n_out ? n_lo + out_per_block : n_out;
    if (k_in >= 256) {
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        for (int n = n_lo + wave; n < n_hi; n += 4) {
            const float* wr = w + (int64_t)n * k_in;
            float acc[TOK];
#pragma unroll
            for (int tt = 0; tt < TOK; ++tt) acc[tt] = 0.f;
            for (int k = lane; k < k_in; k += 64) {
                const float wv = wr[k];
#pragma unroll
                for (int tt = 0; tt < TOK; ++tt) acc[tt] += wv * xs[tt * k_in + k];
            }
#pragma unroll
            for (int tt = 0; tt < TOK; ++tt) {
                const float sum = wave_sum(acc[tt]);
                if (lane == 0 && tt < nt) out[(t0 + tt) * n_out + n] = sum;
            }
        }
    } else {
        for (int n = n_lo + threadIdx.x; n < n_hi; n += 256) {
            const float* wr = w + (int64_t)n * k_in;
            float acc[TOK];
#pragma unroll
            for (int tt = 0; tt < TOK; ++tt) acc[tt] = 0.f;
            for (int k = 0; k < k_in; ++k) {
                const float wv = wr[k];
#pragma unroll
                for (int tt = 0; tt < TOK; ++tt) acc[tt] += wv * xs[tt * k_in + k];
            }
#pragma unroll
            for (int tt = 0; tt < TOK; ++tt)
                if (tt < nt) out[(t0 + tt) * n_out + n] = acc[tt];
        }
    }
}

}  // namespace NVX_NS

using namespace NVX_NS;

extern "C" int nvx_skinny_proj(const void* x, int64_t x_stride, int fmt, const float* w, int in_act, float* out, int64_t n_tok,
                               int64_t n_out, int64_t k_in, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && (in_act == 0 || in_act == 1), NVX_EINVAL, "nvx_skinny_proj: fmt must be 0..2, in_act 0 or 1");
    NVX_REQUIRE(n_tok >= 0 && n_out > 0 && n_out < (1 << 24) && k_in > 0 && k_in <= 12288 && x_stride >= k_in, NVX_EINVAL,
                "nvx_skinny_proj: bad sizes (at most 12288 inputs)");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && w && out, NVX_EINVAL, "nvx_skinny_proj: null pointer");
    // the outputs are split over workgroups too (8 a workgroup for wide inputs, 256 for narrow ones): a step of few tokens would
    // otherwise be a handful of workgroups walking all outputs one after another
    const int opb = k_in >= 256 ? 8 : 256;
    const int64_t chunks = (n_out + opb - 1) / opb;
    NVX_REQUIRE(chunks <= 65535, NVX_EINVAL, "nvx_skinny_proj: too many outputs");
    if (k_in <= 3072) {
        const int64_t blocks = (n_tok + 3) / 4;
        NVX_REQUIRE(blocks < (1ll << 31), NVX_EINVAL, "nvx_skinny_proj: too many tokens");
        NVX_FMT_CALL(fmt, hipLaunchKernelGGL((skinny_proj_kernel<A_, 4>), dim3((unsigned)blocks, (unsigned)chunks), dim3(256),
                                             (size_t)(4 * k_in) * sizeof(float), (hipStream_t)stream, (const A_*)x, x_stride, w, in_act, out, n_tok,
                                             (int)n_out, (int)k_in, opb));
    } else {
        NVX_REQUIRE(n_tok < (1ll << 31), NVX_EINVAL, "nvx_skinny_proj: too many tokens");
        NVX_FMT_CALL(fmt, hipLaunchKernelGGL((skinny_proj_kernel<A_, 1>), dim3((unsigned)n_tok, (unsigned)chunks), dim3(256),
                                             (size_t)k_in * sizeof(float), (hipStream_t)stream, (const A_*)x, x_stride, w, in_act, out, n_tok,
                                             (int)n_out, (int)k_in, opb));
    }
    return nvx_check_launch("nvx_skinny_proj");
}

extern "C" int nvx_gated_residual_norm(const void* y, int64_t y_stride, const void* y2, int64_t y2_stride, const float* w_y,
                                       const float* w_y2, const void* gate, int64_t gate_stride, const float* gate_bias, int fmt,
                                       float mult, float* x, const float* w_norm, int groups, float eps, void* h_out, int64_t n_tok,
                                       int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_gated_residual_norm: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && width > 0 && width < (1 << 30) && groups >= 1 && width % groups == 0, NVX_EINVAL,
                "nvx_gated_residual_norm: bad sizes (the width must be a multiple of the groups)");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && (y || w_norm), NVX_EINVAL, "nvx_gated_residual_norm: null pointer");
    NVX_REQUIRE(!y || y_stride >= width, NVX_EINVAL, "nvx_gated_residual_norm: row stride of y");
    NVX_REQUIRE(!y2 || (y && w_y && w_y2 && y2_stride >= width), NVX_EINVAL, "nvx_gated_residual_norm: two branches need both weights");
    NVX_REQUIRE(!gate || (y && gate_stride >= width), NVX_EINVAL, "nvx_gated_residual_norm: a gate needs a result to gate");
    NVX_REQUIRE(!w_norm || h_out, NVX_EINVAL, "nvx_gated_residual_norm: the norm needs an output");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(gated_residual_norm_kernel<A_>, dim3((unsigned)n_tok), dim3(256), 0, (hipStream_t)stream,
                                         (const A_*)y, y_stride, (const A_*)y2, y2_stride, w_y, w_y2, (const A_*)gate, gate_stride,
                                         gate_bias, mult, x, w_norm, groups, eps, (A_*)h_out, (int)width));
    return nvx_check_launch("nvx_gated_residual_norm");
}

extern "C" int nvx_head_norm_gate(const float* o, const float* w, int w_shared, const void* gate, int64_t gate_stride, int kind, int fmt,
                                  float eps, void* out, int64_t n_tok, int64_t heads, int64_t vdim, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && kind >= 0 && kind <= 2, NVX_EINVAL, "nvx_head_norm_gate: fmt must be 0..2, kind 0..2");
    NVX_REQUIRE(n_tok >= 0 && heads > 0 && vdim > 0 && heads * vdim < (1 << 30), NVX_EINVAL, "nvx_head_norm_gate: bad sizes");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(o && w && out && (kind == 0 || (gate && gate_stride >= heads * vdim)), NVX_EINVAL, "nvx_head_norm_gate: null pointer");
    const int64_t rows = n_tok * heads;
    NVX_REQUIRE((rows + 3) / 4 < (1ll << 31), NVX_EINVAL, "nvx_head_norm_gate: too many rows");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(head_norm_gate_kernel<A_>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream, o, w,
                                         w_shared, (const A_*)gate, gate_stride, kind, eps, (A_*)out, rows, (int)heads, (int)vdim));
    return nvx_check_launch("nvx_head_norm_gate");
}

extern "C" int nvx_postnorm_residual(const void* y, int64_t y_stride, const void* y2, int64_t y2_stride, float a, float b, const float* w_post,
                                     int64_t w_post_n, int fmt, float* x, const float* w_next, int64_t w_next_n, float eps, void* h_out,
                                     int64_t n_tok, int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_postnorm_residual: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && width > 0 && width < (1 << 30), NVX_EINVAL, "nvx_postnorm_residual: bad sizes");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x && (y || h_out), NVX_EINVAL, "nvx_postnorm_residual: null pointer");
    NVX_REQUIRE(!y || (y_stride >= width && w_post && (w_post_n == 1 || w_post_n == width)), NVX_EINVAL,
                "nvx_postnorm_residual: a result needs its norm weight (one number or one per channel)");
    NVX_REQUIRE(!y2 || (y && y2_stride >= width), NVX_EINVAL, "nvx_postnorm_residual: a second result needs a first");
    NVX_REQUIRE(!w_next || (h_out && (w_next_n == 1 || w_next_n == width)), NVX_EINVAL, "nvx_postnorm_residual: the closing norm needs an output");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(postnorm_residual_kernel<A_>, dim3((unsigned)n_tok), dim3(256), 0, (hipStream_t)stream, (const A_*)y,
                                         y_stride, (const A_*)y2, y2_stride, a, b, w_post, (int)w_post_n, x, w_next, (int)w_next_n, eps, (A_*)h_out,
                                         (int)width));
    return nvx_check_launch("nvx_postnorm_residual");
}

extern "C" int nvx_hyper_mix(const float* x_in, int64_t in_tok_stride, int64_t in_stream_stride, const void* y, int64_t y_stride, int fmt,
                             const float* scale, const float* mix, const float* w_out, const float* w_in, const float* w_norm, float eps,
                             float* x_out, void* h_out, int64_t n_tok, int64_t n_streams, int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_hyper_mix: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_streams >= 1 && n_streams <= 16 && width > 0, NVX_EINVAL, "nvx_hyper_mix: bad sizes (at most 16 streams)");
    NVX_REQUIRE(width <= 15360, NVX_EUNSUPPORTED, "nvx_hyper_mix: a row must fit LDS as float32 (width <= 15360)");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(x_in && x_out, NVX_EINVAL, "nvx_hyper_mix: null pointer");
    NVX_REQUIRE(in_tok_stride >= width && (in_stream_stride == 0 || in_stream_stride >= width), NVX_EINVAL, "nvx_hyper_mix: strides of the streams");
    NVX_REQUIRE(!y || (y_stride >= width && mix && w_out), NVX_EINVAL, "nvx_hyper_mix: a result needs the mixing matrix and its output weights");
    NVX_REQUIRE(x_in != x_out || (in_tok_stride == n_streams * width && in_stream_stride == width), NVX_EINVAL,
                "nvx_hyper_mix: streams updated in place keep their layout");
    const size_t lds = (size_t)width * sizeof(float);
#define NVX_HYPER(MAXS)                                                                                                               \
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL((hyper_mix_kernel<A_, MAXS>), dim3((unsigned)n_tok), dim3(256), lds, (hipStream_t)stream, x_in, \
                                         in_tok_stride, in_stream_stride, (const A_*)y, y_stride, scale, mix, w_out, w_in, w_norm, eps, \
                                         x_out, (A_*)h_out, (int)n_streams, (int)width))
    if (n_streams <= 1) NVX_HYPER(1);
    else if (n_streams <= 2) NVX_HYPER(2);
    else if (n_streams <= 4) NVX_HYPER(4);
    else if (n_streams <= 8) NVX_HYPER(8);
    else NVX_HYPER(16);
#undef NVX_HYPER
    return nvx_check_launch("nvx_hyper_mix");
}

extern "C" int nvx_embed_scale(const int64_t* ids, const void* table, int fmt, int64_t vocab, float scale, float* x, void* h, int64_t n_tok,
                               int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && n_tok >= 0 && vocab > 0 && width > 0 && width < (1 << 30), NVX_EINVAL, "nvx_embed_scale: bad arguments");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(ids && table && x, NVX_EINVAL, "nvx_embed_scale: null pointer");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(embed_scale_kernel<A_>, dim3((unsigned)n_tok), dim3(256), 0, (hipStream_t)stream, ids, (const A_*)table, vocab,
                                         scale, x, (A_*)h, (int)width));
    return nvx_check_launch("nvx_embed_scale");
}

extern "C" int nvx_tanh_cap(const void* in, int fmt, float cap, float* out, int64_t n, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && n >= 0, NVX_EINVAL, "nvx_tanh_cap: bad arguments");
    if (n == 0) return NVX_OK;
    NVX_REQUIRE(in && out, NVX_EINVAL, "nvx_tanh_cap: null pointer");
    int64_t blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(tanh_cap_kernel<A_>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const A_*)in, cap, out, n));
    return nvx_check_launch("nvx_tanh_cap");
}
