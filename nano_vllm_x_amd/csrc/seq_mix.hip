// Kernels of layer stacks that keep a 32-bit residual stream and per-sequence recurrent state:
//   - boundary norm: post-norm of a sublayer's output + residual add (+ weighted sum over the results of all layers so
//     far) + pre-norm of the next sublayer, one launch per sublayer boundary;
//   - short causal convolution over time on every channel ("canon"), its tail of inputs kept per sequence;
//   - gated linear recurrence with state-independent gates (minGRU);
//   - squared ReLU.
// Activations (`fmt`: 0 bfloat16, 1 float16, 2 float32) are what the matrix products read and write; norm weights,
// convolution taps, mixing weights, the residual stream and every state are float32 in all formats.
// A batch is a ragged list of sequences: tokens [qo_indptr[b], qo_indptr[b+1]) belong to sequence b, whose first token
// of this step stands at position pos0[b] and whose state lives in slot state_slot[b] (a negative slot: a padding row,
// nothing is read or written).  A sequence at position 0 has no state yet: the kernels take zeros instead of reading it,
// so a slot needs no clearing when it is handed to a new sequence.
#include "nvx_dev.h"

namespace NVX_NS {

template <typename A> __device__ __forceinline__ float ldf(const A* p, int64_t i) { return (float)p[i]; }
template <typename A> __device__ __forceinline__ void stf(A* p, int64_t i, float v) { p[i] = (A)v; }

// four consecutive elements at once (the caller guarantees a multiple-of-4 offset into a 16-byte-aligned row)
typedef float f32x4v __attribute__((ext_vector_type(4)));
template <typename A> struct vec4 { typedef A type __attribute__((ext_vector_type(4))); };
template <typename A> __device__ __forceinline__ f32x4v ld4(const A* p) {
    return __builtin_convertvector(*reinterpret_cast<const typename vec4<A>::type*>(p), f32x4v);
}
template <typename A> __device__ __forceinline__ void st4(A* p, f32x4v v) {
    *reinterpret_cast<typename vec4<A>::type*>(p) = __builtin_convertvector(v, typename vec4<A>::type);
}

// sum over a workgroup of 256 threads; every thread gets the total.  `red` holds 4 floats; safe to call repeatedly.
__device__ __forceinline__ float block_sum256(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();                       // the previous call's readers are done
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// ---- boundary norm ------------------------------------------------------------------------------------------------
// Per token t (one workgroup each):
//   r   = res[t] + m[t] / rms(m[t]) * (1 + w_post)                 (res == null: r = the normed m alone)
//   hist[hist_slot][t] = r                                          (hist_slot >= 0)
//   x   = sum_{j < n_mix} mix[j] * hist[j][t]                       (n_mix > 0; hist[hist_slot] is r), else x = r
//   x_out[t] = x
//   y   = x / rms(x) * (1 + w_pre)  ->  y_f32[t] (float) or y_act[t] (activation format), whichever is given
template <typename A>
__global__ __launch_bounds__(256) void boundary_norm_kernel(
    const A* __restrict__ m, int64_t m_stride, const float* __restrict__ res, const float* __restrict__ w_post,
    float* __restrict__ hist, int64_t hist_stride, int hist_slot, int n_mix, const float* __restrict__ mix,
    float* __restrict__ x_out, const float* __restrict__ w_pre, float* __restrict__ y_f32, A* __restrict__ y_act,
    int width, float eps) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const A* mr = m + t * m_stride;
    const int64_t row = t * (int64_t)width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) { const float v = ldf(mr, c); ss += v * v; }
    const float r_post = 1.0f / sqrtf(block_sum256(ss, red) / (float)width + eps);
    float ss2 = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
        float r = ldf(mr, c) * r_post * (1.0f + w_post[c]);
        if (res) r += res[row + c];
        if (hist_slot >= 0) hist[(int64_t)hist_slot * hist_stride + row + c] = r;
        float x = r;
        if (n_mix > 0) {
            x = 0.f;
            for (int j = 0; j < n_mix; ++j)
                x += mix[j] * (j == hist_slot ? r : hist[(int64_t)j * hist_stride + row + c]);
        }
        x_out[row + c] = x;
        ss2 += x * x;
    }
    if (!w_pre) return;
    const float r_pre = 1.0f / sqrtf(block_sum256(ss2, red) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += 256) {
        const float y = x_out[row + c] * r_pre * (1.0f + w_pre[c]);   // this thread's own store, read back
        if (y_f32) y_f32[row + c] = y;
        else stf(y_act, row + c, y);
    }
}

// The same, for rows of at most 256 * 4 * VPT values with a multiple of 4 of them: every thread keeps its part of the row
// in registers, so m and the stream are read once and written once.
template <typename A, int VPT>
__global__ __launch_bounds__(256) void boundary_norm_reg_kernel(
    const A* __restrict__ m, int64_t m_stride, const float* __restrict__ res, const float* __restrict__ w_post,
    float* __restrict__ hist, int64_t hist_stride, int hist_slot, int n_mix, const float* __restrict__ mix,
    float* __restrict__ x_out, const float* __restrict__ w_pre, float* __restrict__ y_f32, A* __restrict__ y_act,
    int width, float eps, const float* __restrict__ taps, int taps_n, float* __restrict__ state, const int64_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slot) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const A* mr = m + t * m_stride;
    const int64_t row = t * (int64_t)width;
    f32x4v v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int c = (threadIdx.x + k * 256) * 4;
        v[k] = c < width ? ld4(mr + c) : f32x4v{0.f, 0.f, 0.f, 0.f};
        ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
    }
    const float r_post = 1.0f / sqrtf(block_sum256(ss, red) / (float)width + eps);
    float ss2 = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int c = (threadIdx.x + k * 256) * 4;
        if (c >= width) continue;
        f32x4v r = v[k] * r_post * (1.0f + *reinterpret_cast<const f32x4v*>(w_post + c));
        if (res) r += *reinterpret_cast<const f32x4v*>(res + row + c);
        if (hist_slot >= 0) *reinterpret_cast<f32x4v*>(hist + (int64_t)hist_slot * hist_stride + row + c) = r;
        f32x4v x = r;
        if (n_mix > 0) {
            x = f32x4v{0.f, 0.f, 0.f, 0.f};
            for (int j = 0; j < n_mix; ++j)
                x += mix[j] * (j == hist_slot ? r : *reinterpret_cast<const f32x4v*>(hist + (int64_t)j * hist_stride + row + c));
        }
        *reinterpret_cast<f32x4v*>(x_out + row + c) = x;
        v[k] = x;
        ss2 += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
    if (!w_pre) return;
    const float r_pre = 1.0f / sqrtf(block_sum256(ss2, red) / (float)width + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int c = (threadIdx.x + k * 256) * 4;
        if (c >= width) continue;
        const f32x4v y = v[k] * r_pre * (1.0f + *reinterpret_cast<const f32x4v*>(w_pre + c));
        if (taps) {
            // one token per sequence: the convolution over the sequence's tail and the tail's shift happen here, in the one
            // workgroup that touches this sequence (a thread reads and writes only its own channels)
            const int slot = state_slot[t];
            if (slot < 0) { st4(y_act + row + c, f32x4v{0.f, 0.f, 0.f, 0.f}); continue; }
            const int hist_n = taps_n - 1;
            const bool had = pos0[t] > 0;
            f32x4v acc = y + *reinterpret_cast<const f32x4v*>(taps + (int64_t)hist_n * width + c) * y;
            float* st = state + (int64_t)slot * hist_n * width + c;
            for (int r = 0; r < hist_n; ++r) {
                const f32x4v old = had ? *reinterpret_cast<const f32x4v*>(st + (int64_t)r * width) : f32x4v{0.f, 0.f, 0.f, 0.f};
                acc += *reinterpret_cast<const f32x4v*>(taps + (int64_t)r * width + c) * old;
                if (r > 0) *reinterpret_cast<f32x4v*>(st + (int64_t)(r - 1) * width) = old;
            }
            if (hist_n > 0) *reinterpret_cast<f32x4v*>(st + (int64_t)(hist_n - 1) * width) = y;
            st4(y_act + row + c, acc);
        } else if (y_f32) *reinterpret_cast<f32x4v*>(y_f32 + row + c) = y;
        else st4(y_act + row + c, y);
    }
}

// ---- canon: h + causal convolution over time, per channel -----------------------------------------------------------
// taps[j][c] (taps_n rows of `width`) multiplies channel c of the input (taps_n - 1 - j) tokens back.  state[slot][r] (r < taps_n - 1) is the input at position
// pos0 - (taps_n - 1) + r.
template <typename A>
__global__ __launch_bounds__(256) void canon_conv_kernel(
    const float* __restrict__ h, const float* __restrict__ taps, int taps_n, const float* __restrict__ state,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slot, A* __restrict__ out, int64_t n_tok, int width) {
    const int64_t total = n_tok * (int64_t)width;
    for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
        const int64_t t = id / width;
        const int c = (int)(id - t * width);
        const int b = tok_seq ? tok_seq[t] : (int)t;
        const int slot = state_slot[b];
        if (slot < 0) { stf(out, id, 0.f); continue; }
        const int64_t q0 = qo_indptr ? qo_indptr[b] : t;
        const int64_t local = t - q0;
        const bool has_state = pos0[b] > 0;
        const int hist_n = taps_n - 1;
        float acc = h[id];
        for (int j = 0; j < taps_n; ++j) {
            const int64_t s = local - hist_n + j;
            float v;
            if (s >= 0) v = h[(q0 + s) * width + c];
            else v = has_state ? state[((int64_t)slot * hist_n + (hist_n + s)) * width + c] : 0.f;
            acc += taps[(int64_t)j * width + c] * v;
        }
        stf(out, id, acc);
    }
}

// The same with four channels per thread (width a multiple of 4): workgroup (x, t) takes 1024 channels of token t.
template <typename A>
__global__ __launch_bounds__(256) void canon_conv_vec_kernel(
    const float* __restrict__ h, const float* __restrict__ taps, int taps_n, const float* __restrict__ state,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slot, A* __restrict__ out, int width) {
    const int64_t t = blockIdx.y;
    const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= width) return;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const int slot = state_slot[b];
    if (slot < 0) { st4(out + t * width + c, f32x4v{0.f, 0.f, 0.f, 0.f}); return; }
    const int64_t q0 = qo_indptr ? qo_indptr[b] : t;
    const int64_t local = t - q0;
    const bool has_state = pos0[b] > 0;
    const int hist_n = taps_n - 1;
    f32x4v acc = *reinterpret_cast<const f32x4v*>(h + t * width + c);
    for (int j = 0; j < taps_n; ++j) {
        const int64_t s = local - hist_n + j;
        f32x4v v;
        if (s >= 0) v = *reinterpret_cast<const f32x4v*>(h + (q0 + s) * width + c);
        else if (has_state) v = *reinterpret_cast<const f32x4v*>(state + ((int64_t)slot * hist_n + (hist_n + s)) * width + c);
        else continue;
        acc += *reinterpret_cast<const f32x4v*>(taps + (int64_t)j * width + c) * v;
    }
    st4(out + t * width + c, acc);
}

// After the convolution has read the old tail: the last taps_n - 1 inputs of every sequence become its new tail.
__global__ __launch_bounds__(256) void canon_state_kernel(
    const float* __restrict__ h, int taps_n, float* __restrict__ state, const int32_t* __restrict__ qo_indptr,
    const int64_t* __restrict__ pos0, const int32_t* __restrict__ state_slot, int width) {
    const int b = blockIdx.y;
    const int slot = state_slot[b];
    if (slot < 0) return;
    const int64_t q0 = qo_indptr ? qo_indptr[b] : b;
    const int64_t n = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
    if (n <= 0) return;
    const bool has_state = pos0[b] > 0;
    const int hist_n = taps_n - 1;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < width; c += gridDim.x * 256) {
        float* st = state + (int64_t)slot * hist_n * width + c;
        for (int r = 0; r < hist_n; ++r) {        // ascending: row r takes old row r + n, which is not yet overwritten
            const int64_t s = n - hist_n + r;
            float v;
            if (s >= 0) v = h[(q0 + s) * width + c];
            else v = has_state ? st[(int64_t)(r + n) * width] : 0.f;
            st[(int64_t)r * width] = v;
        }
    }
}

// ---- squared ReLU ---------------------------------------------------------------------------------------------------
template <typename A>
__global__ __launch_bounds__(256) void relu2_kernel(const A* __restrict__ x, A* __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const float v = fmaxf(ldf(x, i), 0.f);
        stf(y, i, v * v);
    }
}

// 16-bit formats, eight entries per thread as one 16-byte load and store (n8 = n / 8)
template <typename A>
__global__ __launch_bounds__(256) void relu2_vec8_kernel(const A* __restrict__ x, A* __restrict__ y, int64_t n8) {
    union Pack { uint4 v; A a[8]; };
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        Pack in, out;
        in.v = reinterpret_cast<const uint4*>(x)[i];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float v = fmaxf((float)in.a[k], 0.f);
            out.a[k] = (A)(v * v);
        }
        reinterpret_cast<uint4*>(y)[i] = out.v;
    }
}

// ---- minGRU ---------------------------------------------------------------------------------------------------------
// zxg[t] = [ z pre-activation | candidate pre-activation u | output-gate pre-activation g ], `width` each.
//   z = sigmoid(.),  cand = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),  S <- (1 - z) S + z cand,  out = S * silu(g)
// The recurrence is S_t = a_t S_(t-1) + b_t with a = 1 - z, b = z cand: segments of the time axis are scanned in parallel
// and chained.  All of it in float32.
__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }
// 16-bit activation formats: the hardware exponential (relative error ~1e-6, far below the format's own rounding)
template <typename A> __device__ __forceinline__ float sigm(float v) {
    if constexpr (sizeof(A) == 4) return 1.0f / (1.0f + expf(-v));
    else return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
}

// A workgroup takes GRU_CB channels of one sequence and walks its tokens in rounds of GRU_NSEG * SEG tokens: thread
// (segment, channel pair) scans SEG consecutive tokens from a zero state, keeping the running product of a; the segments'
// results are chained through LDS, and every thread then adds its incoming state times the running product.
#define GRU_CB 32        // channels per workgroup (16 lanes x 2)
#define GRU_NSEG 16      // time segments per round

template <typename A, int SEG>
__global__ __launch_bounds__(256) void mingru_scan_kernel(
    const A* __restrict__ zxg, int64_t row_stride, float* __restrict__ state, const int32_t* __restrict__ qo_indptr,
    const int64_t* __restrict__ pos0, const int32_t* __restrict__ state_slot, A* __restrict__ out, int width) {
    __shared__ float agg_a[GRU_NSEG][GRU_CB], agg_b[GRU_NSEG][GRU_CB];
    const int b = blockIdx.y;
    const int slot = state_slot[b];
    if (slot < 0) return;
    const int64_t q0 = qo_indptr ? qo_indptr[b] : b;
    const int64_t n = qo_indptr ? qo_indptr[b + 1] - q0 : 1;
    if (n <= 0) return;
    const int seg = threadIdx.x >> 4, cl = (threadIdx.x & 15) * 2;
    const int c = blockIdx.x * GRU_CB + cl;
    const bool live0 = c < width, live1 = c + 1 < width;
    const bool had = pos0[b] > 0;
    // the pair can be moved as one value when both channels exist and every row keeps the pair's alignment
    const bool pair_ok = live1 && width % 2 == 0 && row_stride % 2 == 0 && (reinterpret_cast<uintptr_t>(zxg) % (2 * sizeof(A))) == 0;
    float carry0 = (live0 && had) ? state[(int64_t)slot * width + c] : 0.f;
    float carry1 = (live1 && had) ? state[(int64_t)slot * width + c + 1] : 0.f;
    for (int64_t base = 0; base < n; base += SEG * GRU_NSEG) {
        const int64_t t0 = base + (int64_t)seg * SEG;
        float pa0[SEG], ps0[SEG], gg0[SEG], pa1[SEG], ps1[SEG], gg1[SEG];
        float a0 = 1.f, s0 = 0.f, a1 = 1.f, s1 = 0.f;
#pragma unroll
        for (int i = 0; i < SEG; ++i) {
            const int64_t t = t0 + i;
            gg0[i] = gg1[i] = 0.f;
            if (t < n) {
                const A* r = zxg + (q0 + t) * row_stride;
                float zz[2], uu[2], gq[2];
                if (pair_ok) {             // both channels with one load each (the pair is aligned to its own size)
                    typedef A a2 __attribute__((ext_vector_type(2)));
                    const a2 zv = *reinterpret_cast<const a2*>(r + c), uv = *reinterpret_cast<const a2*>(r + width + c),
                             gv = *reinterpret_cast<const a2*>(r + 2 * (int64_t)width + c);
                    zz[0] = (float)zv.x; zz[1] = (float)zv.y; uu[0] = (float)uv.x; uu[1] = (float)uv.y; gq[0] = (float)gv.x; gq[1] = (float)gv.y;
                } else {
                    zz[0] = live0 ? ldf(r, c) : 0.f; uu[0] = live0 ? ldf(r, (int64_t)width + c) : 0.f; gq[0] = live0 ? ldf(r, 2 * (int64_t)width + c) : 0.f;
                    zz[1] = live1 ? ldf(r, c + 1) : 0.f; uu[1] = live1 ? ldf(r, (int64_t)width + c + 1) : 0.f;
                    gq[1] = live1 ? ldf(r, 2 * (int64_t)width + c + 1) : 0.f;
                }
                {
                    const float z = sigm<A>(zz[0]);
                    const float cand = uu[0] >= 0.f ? uu[0] + 0.5f : sigm<A>(uu[0]);
                    gg0[i] = gq[0] * sigm<A>(gq[0]);
                    s0 = (1.0f - z) * s0 + z * cand;
                    a0 *= (1.0f - z);
                }
                {
                    const float z = sigm<A>(zz[1]);
                    const float cand = uu[1] >= 0.f ? uu[1] + 0.5f : sigm<A>(uu[1]);
                    gg1[i] = gq[1] * sigm<A>(gq[1]);
                    s1 = (1.0f - z) * s1 + z * cand;
                    a1 *= (1.0f - z);
                }
            }
            pa0[i] = a0; ps0[i] = s0; pa1[i] = a1; ps1[i] = s1;
        }
        __syncthreads();                   // the previous round's readers are done
        agg_a[seg][cl] = a0; agg_b[seg][cl] = s0;
        agg_a[seg][cl + 1] = a1; agg_b[seg][cl + 1] = s1;
        __syncthreads();
        float in0 = carry0, in1 = carry1;  // state before this thread's first token
        for (int k = 0; k < seg; ++k) {
            in0 = agg_a[k][cl] * in0 + agg_b[k][cl];
            in1 = agg_a[k][cl + 1] * in1 + agg_b[k][cl + 1];
        }
        float l0 = in0, l1 = in1;
        for (int k = seg; k < GRU_NSEG; ++k) {
            l0 = agg_a[k][cl] * l0 + agg_b[k][cl];
            l1 = agg_a[k][cl + 1] * l1 + agg_b[k][cl + 1];
        }
        carry0 = l0;                       // state after the round's last token (segments past the end are identities)
        carry1 = l1;
#pragma unroll
        for (int i = 0; i < SEG; ++i) {
            const int64_t t = t0 + i;
            if (t < n) {
                if (live0) stf(out, (q0 + t) * (int64_t)width + c, (pa0[i] * in0 + ps0[i]) * gg0[i]);
                if (live1) stf(out, (q0 + t) * (int64_t)width + c + 1, (pa1[i] * in1 + ps1[i]) * gg1[i]);
            }
        }
    }
    if (seg == 0) {
        if (live0) state[(int64_t)slot * width + c] = carry0;
        if (live1) state[(int64_t)slot * width + c + 1] = carry1;
    }
}

// one token per sequence (a decode step): thread = (sequence, channel)
template <typename A>
__global__ __launch_bounds__(256) void mingru_step_kernel(
    const A* __restrict__ zxg, int64_t row_stride, float* __restrict__ state, const int64_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slot, A* __restrict__ out, int64_t n_seq, int width) {
    const int64_t total = n_seq * (int64_t)width;
    for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
        const int64_t b = id / width;
        const int c = (int)(id - b * width);
        const int slot = state_slot[b];
        if (slot < 0) { stf(out, id, 0.f); continue; }
        const A* r = zxg + b * row_stride;
        const float z = sigm<A>(ldf(r, c));
        const float u = ldf(r, (int64_t)width + c);
        const float cand = u >= 0.f ? u + 0.5f : sigm<A>(u);
        const float g = ldf(r, 2 * (int64_t)width + c);
        float* sp = state + (int64_t)slot * width + c;
        const float s = (1.0f - z) * (pos0[b] > 0 ? *sp : 0.f) + z * cand;
        *sp = s;
        stf(out, id, s * (g * sigm<A>(g)));
    }
}

// ---- real-gated linear recurrent unit ----------------------------------------------------------------------------------
// Per token and channel c (block b = c / block_width, j = c % block_width), all of it float32:
//   r = sigmoid(gates[b][t][j] + gate_bias[c]),  i = sigmoid(gates[b][t][block_width + j] + gate_bias[width + c])
//   log a = -rate[c] * r,  a = exp(log a),  S <- a S + sqrt(1 - a^2) * i * u[t][c],  out = S * gelu_tanh(y[t][c])
// `gates` is what a batched product over the blocks leaves: (blocks, tokens, 2 * block_width), recurrence gate | input gate;
// `rate` is the channel's constant (the design's multiplier times softplus of its parameter).  1 - a^2 is formed as
// -expm1(2 log a), which keeps its leading digits where a is close to one.  The scan is the one of the minGRU kernel:
// S_t = a_t S_(t-1) + b_t by segments of the time axis that are chained through LDS.
struct RglruIn {
    const void* y; int64_t y_stride;
    const void* u; int64_t u_stride;
    const void* gates; int64_t g_block_stride, g_tok_stride;
    const float* gate_bias; const float* rate;
    int block_width, width;
};

__device__ __forceinline__ float gelu_tanh_f(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// (a, b, output gate) of token row `t` (a row of the step) and channel c
template <typename A>
__device__ __forceinline__ void rglru_cell(const RglruIn& in, int64_t t, int c, float& a, float& b, float& g) {
    const int blk = c / in.block_width, j = c - blk * in.block_width;
    const A* gr = (const A*)in.gates + blk * in.g_block_stride + t * in.g_tok_stride;
    const float r = sigm<A>(ldf(gr, j) + in.gate_bias[c]);
    const float i = sigm<A>(ldf(gr, in.block_width + j) + in.gate_bias[in.width + c]);
    const float log_a = -in.rate[c] * r;
    a = expf(log_a);
    b = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f)) * i * ldf((const A*)in.u, t * in.u_stride + c);
    g = gelu_tanh_f(ldf((const A*)in.y, t * in.y_stride + c));
}

template <typename A, int SEG>
__global__ __launch_bounds__(256) void rglru_scan_kernel(RglruIn in, float* __restrict__ state, const int32_t* __restrict__ qo_indptr,
                                                        const int64_t* __restrict__ pos0, const int32_t* __restrict__ state_slot,
                                                        A* __restrict__ out) {
    __shared__ float agg_a[GRU_NSEG][GRU_CB], agg_b[GRU_NSEG][GRU_CB];
    const int b = blockIdx.y;
    const int slot = state_slot[b];
    if (slot < 0) return;
    const int64_t q0 = qo_indptr[b];
    const int64_t n = qo_indptr[b + 1] - q0;
    if (n <= 0) return;
    const int width = in.width;
    const int seg = threadIdx.x >> 4, cl = (threadIdx.x & 15) * 2;
    const int c = blockIdx.x * GRU_CB + cl;
    const bool live[2] = {c < width, c + 1 < width};
    const bool had = pos0[b] > 0;
    float carry[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) carry[k] = (live[k] && had) ? state[(int64_t)slot * width + c + k] : 0.f;
    for (int64_t base = 0; base < n; base += SEG * GRU_NSEG) {
        const int64_t t0 = base + (int64_t)seg * SEG;
        float pa[2][SEG], ps[2][SEG], gg[2][SEG];
        float ar[2] = {1.f, 1.f}, sr[2] = {0.f, 0.f};
#pragma unroll
        for (int i = 0; i < SEG; ++i) {
            const int64_t t = t0 + i;
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                gg[k][i] = 0.f;
                if (t < n && live[k]) {
                    float a, bb, g;
                    rglru_cell<A>(in, q0 + t, c + k, a, bb, g);
                    sr[k] = a * sr[k] + bb;
                    ar[k] *= a;
                    gg[k][i] = g;
                }
                pa[k][i] = ar[k];
                ps[k][i] = sr[k];
            }
        }
        __syncthreads();                   // the previous round's readers are done
#pragma unroll
        for (int k = 0; k < 2; ++k) { agg_a[seg][cl + k] = ar[k]; agg_b[seg][cl + k] = sr[k]; }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            float in_s = carry[k];         // state before this thread's first token
            for (int q = 0; q < seg; ++q) in_s = agg_a[q][cl + k] * in_s + agg_b[q][cl + k];
            float last = in_s;
            for (int q = seg; q < GRU_NSEG; ++q) last = agg_a[q][cl + k] * last + agg_b[q][cl + k];
            carry[k] = last;               // state after the round's last token (segments past the end are identities)
            if (live[k]) {
#pragma unroll
                for (int i = 0; i < SEG; ++i) {
                    const int64_t t = t0 + i;
                    if (t < n) stf(out, (q0 + t) * (int64_t)width + c + k, (pa[k][i] * in_s + ps[k][i]) * gg[k][i]);
                }
            }
        }
    }
    if (seg == 0) {
#pragma unroll
        for (int k = 0; k < 2; ++k) if (live[k]) state[(int64_t)slot * width + c + k] = carry[k];
    }
}

// one token per sequence (a decode step): thread = (sequence, channel)
template <typename A>
__global__ __launch_bounds__(256) void rglru_step_kernel(RglruIn in, float* __restrict__ state, const int64_t* __restrict__ pos0,
                                                        const int32_t* __restrict__ state_slot, A* __restrict__ out, int64_t n_seq) {
    const int width = in.width;
    const int64_t total = n_seq * (int64_t)width;
    for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
        const int64_t b = id / width;
        const int c = (int)(id - b * width);
        const int slot = state_slot[b];
        if (slot < 0) { stf(out, id, 0.f); continue; }
        float a, bb, g;
        rglru_cell<A>(in, b, c, a, bb, g);
        float* sp = state + (int64_t)slot * width + c;
        const float s = a * (pos0[b] > 0 ? *sp : 0.f) + bb;
        *sp = s;
        stf(out, id, s * g);
    }
}

template <typename A>
static int launch_boundary(const void* m, int64_t m_stride, const float* res, const float* w_post, float* hist, int64_t hist_stride,
                           int hist_slot, int n_mix, const float* mix, float* x_out, const float* w_pre, float* y_f32, void* y_act,
                           int64_t n_tok, int width, float eps, const float* taps, int taps_n, float* state, const int64_t* pos0,
                           const int32_t* state_slot, hipStream_t s) {
    const bool vec = width % 4 == 0 && m_stride % 4 == 0 && hist_stride % 4 == 0 && nvx_aligned16(m) && nvx_aligned16(res) &&
                     nvx_aligned16(w_post) && nvx_aligned16(hist) && nvx_aligned16(x_out) && nvx_aligned16(w_pre) && nvx_aligned16(y_f32) &&
                     nvx_aligned16(y_act) && nvx_aligned16(taps) && nvx_aligned16(state);
    if (taps && !(vec && width <= 8192)) return 1;     // the fused step exists in the register kernel only
#define NVX_BOUNDARY_REG(VPT)                                                                                                         \
    hipLaunchKernelGGL((boundary_norm_reg_kernel<A, VPT>), dim3((unsigned)n_tok), dim3(256), 0, s, (const A*)m, m_stride, res, w_post, \
                       hist, hist_stride, hist_slot, n_mix, mix, x_out, w_pre, y_f32, (A*)y_act, width, eps, taps, taps_n, state, pos0, \
                       state_slot)
    if (vec && width <= 1024) NVX_BOUNDARY_REG(1);
    else if (vec && width <= 2048) NVX_BOUNDARY_REG(2);
    else if (vec && width <= 4096) NVX_BOUNDARY_REG(4);
    else if (vec && width <= 8192) NVX_BOUNDARY_REG(8);
    else
        hipLaunchKernelGGL(boundary_norm_kernel<A>, dim3((unsigned)n_tok), dim3(256), 0, s, (const A*)m, m_stride, res, w_post, hist,
                           hist_stride, hist_slot, n_mix, mix, x_out, w_pre, y_f32, (A*)y_act, width, eps);
#undef NVX_BOUNDARY_REG
    return 0;
}

template <typename A>
static void launch_canon(const float* h, const float* taps, int taps_n, float* state, const int32_t* tok_seq, const int32_t* qo_indptr,
                         const int64_t* pos0, const int32_t* state_slot, void* out, int64_t n_tok, int64_t n_seq, int width,
                         hipStream_t s) {
    if (width % 4 == 0 && n_tok <= 65535 && nvx_aligned16(h) && nvx_aligned16(state) && nvx_aligned16(out) && nvx_aligned16(taps)) {
        hipLaunchKernelGGL(canon_conv_vec_kernel<A>, dim3((unsigned)((width / 4 + 255) / 256), (unsigned)n_tok), dim3(256), 0, s, h, taps,
                           taps_n, (const float*)state, tok_seq, qo_indptr, pos0, state_slot, (A*)out, width);
    } else {
        int64_t blocks = (n_tok * width + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        hipLaunchKernelGGL(canon_conv_kernel<A>, dim3((unsigned)blocks), dim3(256), 0, s, h, taps, taps_n, (const float*)state, tok_seq,
                           qo_indptr, pos0, state_slot, (A*)out, n_tok, width);
    }
    if (taps_n > 1)
        hipLaunchKernelGGL(canon_state_kernel, dim3((unsigned)((width + 255) / 256), (unsigned)n_seq), dim3(256), 0, s, h, taps_n, state,
                           qo_indptr, pos0, state_slot, width);
}

template <typename A>
static void launch_mingru(const void* zxg, int64_t row_stride, float* state, const int32_t* qo_indptr, const int64_t* pos0,
                          const int32_t* state_slot, void* out, int64_t n_seq, int width, hipStream_t s) {
    if (!qo_indptr) {
        int64_t blocks = (n_seq * width + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        hipLaunchKernelGGL(mingru_step_kernel<A>, dim3((unsigned)blocks), dim3(256), 0, s, (const A*)zxg, row_stride, state, pos0,
                           state_slot, (A*)out, n_seq, width);
        return;
    }
    hipLaunchKernelGGL((mingru_scan_kernel<A, 8>), dim3((unsigned)((width + GRU_CB - 1) / GRU_CB), (unsigned)n_seq), dim3(256), 0, s, (const A*)zxg,
                       row_stride, state, qo_indptr, pos0, state_slot, (A*)out, width);
}

template <typename A>
static void launch_rglru(const RglruIn& in, float* state, const int32_t* qo_indptr, const int64_t* pos0, const int32_t* state_slot, void* out,
                         int64_t n_seq, hipStream_t s) {
    if (!qo_indptr) {
        int64_t blocks = (n_seq * in.width + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        hipLaunchKernelGGL(rglru_step_kernel<A>, dim3((unsigned)blocks), dim3(256), 0, s, in, state, pos0, state_slot, (A*)out, n_seq);
        return;
    }
    hipLaunchKernelGGL((rglru_scan_kernel<A, 8>), dim3((unsigned)((in.width + GRU_CB - 1) / GRU_CB), (unsigned)n_seq), dim3(256), 0, s, in, state,
                       qo_indptr, pos0, state_slot, (A*)out);
}

}  // namespace NVX_NS

using namespace NVX_NS;

#define NVX_FMT_DISPATCH(fmt, CALL)                                         \
    do {                                                                    \
        if ((fmt) == 0) { typedef __bf16 A_; CALL; }                        \
        else if ((fmt) == 1) { typedef _Float16 A_; CALL; }                 \
        else { typedef float A_; CALL; }                                    \
    } while (0)

extern "C" int nvx_boundary_norm(const void* m, int64_t m_row_stride, int fmt, const float* res, const float* w_post, float* hist,
                                 int64_t hist_stride, int hist_slot, int n_mix, const float* mix, float* x_out, const float* w_pre,
                                 float* y_f32, void* y_act, int64_t n_tok, int64_t width, float eps, const float* taps, int taps_n,
                                 float* state, int64_t n_slots, const int64_t* pos0, const int32_t* state_slot, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_boundary_norm: fmt must be 0 (bfloat16), 1 (float16) or 2 (float32)");
    NVX_REQUIRE(n_tok >= 0 && width > 0 && width < (1 << 30) && m_row_stride >= width, NVX_EINVAL, "nvx_boundary_norm: bad sizes");
    if (n_tok == 0) return NVX_OK;
    NVX_REQUIRE(m && w_post && x_out, NVX_EINVAL, "nvx_boundary_norm: null pointer");
    NVX_REQUIRE(hist_slot < 0 || hist, NVX_EINVAL, "nvx_boundary_norm: hist_slot without a history buffer");
    NVX_REQUIRE(n_mix == 0 || (hist && mix && hist_slot >= 0 && hist_slot < n_mix), NVX_EINVAL,
                "nvx_boundary_norm: mixing needs the history buffer, the weights and this result's slot among them");
    NVX_REQUIRE(!hist || hist_stride >= n_tok * width, NVX_EINVAL, "nvx_boundary_norm: history stride smaller than a result");
    NVX_REQUIRE(!w_pre || (y_f32 != nullptr) != (y_act != nullptr), NVX_EINVAL, "nvx_boundary_norm: exactly one output for the pre-norm");
    NVX_REQUIRE(!taps || (w_pre && y_act && !y_f32 && pos0 && state_slot && taps_n >= 1 && taps_n <= 64 && (state || taps_n == 1) && n_slots >= 0),
                NVX_EINVAL, "nvx_boundary_norm: the fused convolution needs the pre-norm, y_act, pos0, state_slot and the state");
    int unfit = 0;
    NVX_FMT_DISPATCH(fmt, unfit = launch_boundary<A_>(m, m_row_stride, res, w_post, hist, hist_stride, hist_slot, n_mix, mix, x_out, w_pre,
                                                      y_f32, y_act, n_tok, (int)width, eps, taps, taps_n, state, pos0, state_slot,
                                                      (hipStream_t)stream));
    NVX_REQUIRE(!unfit, NVX_EUNSUPPORTED, "nvx_boundary_norm: the fused convolution needs a width that is a multiple of 4, at most 8192, "
                                          "and 16-byte aligned tensors");
    return nvx_check_launch("nvx_boundary_norm");
}

extern "C" int nvx_canon_conv(const float* h, const float* taps, int taps_n, float* state, int64_t n_slots, const int32_t* tok_seq,
                              const int32_t* qo_indptr, const int64_t* pos0, const int32_t* state_slot, void* out, int fmt,
                              int64_t n_tok, int64_t n_seq, int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_canon_conv: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_seq >= 0 && n_seq <= 65535 && width > 0 && width < (1 << 30) && taps_n >= 1 && taps_n <= 64 && n_slots >= 0,
                NVX_EINVAL, "nvx_canon_conv: bad sizes");
    if (n_tok == 0 || n_seq == 0) return NVX_OK;
    NVX_REQUIRE(h && taps && out && pos0 && state_slot && (state || taps_n == 1), NVX_EINVAL, "nvx_canon_conv: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_canon_conv: tok_seq and qo_indptr go together");
    NVX_REQUIRE(qo_indptr || n_tok == n_seq, NVX_EINVAL, "nvx_canon_conv: without qo_indptr every sequence has one token");
    NVX_FMT_DISPATCH(fmt, launch_canon<A_>(h, taps, taps_n, state, tok_seq, qo_indptr, pos0, state_slot, out, n_tok, n_seq, (int)width,
                                           (hipStream_t)stream));
    return nvx_check_launch("nvx_canon_conv");
}

extern "C" int nvx_relu2(const void* x, void* y, int fmt, int64_t n, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2 && n >= 0, NVX_EINVAL, "nvx_relu2: bad arguments");
    if (n == 0) return NVX_OK;
    NVX_REQUIRE(x && y, NVX_EINVAL, "nvx_relu2: null pointer");
    if (fmt != 2 && n % 8 == 0 && nvx_aligned16(x) && nvx_aligned16(y)) {
        int64_t blocks = (n / 8 + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        if (fmt == 0)
            hipLaunchKernelGGL(relu2_vec8_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const __bf16*)x, (__bf16*)y, n / 8);
        else
            hipLaunchKernelGGL(relu2_vec8_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const _Float16*)x, (_Float16*)y,
                               n / 8);
        return nvx_check_launch("nvx_relu2");
    }
    int64_t blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    NVX_FMT_DISPATCH(fmt, hipLaunchKernelGGL(relu2_kernel<A_>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const A_*)x,
                                             (A_*)y, n));
    return nvx_check_launch("nvx_relu2");
}

extern "C" int nvx_mingru_scan(const void* zxg, int64_t row_stride, int fmt, float* state, int64_t n_slots, const int32_t* qo_indptr,
                               const int64_t* pos0, const int32_t* state_slot, void* out, int64_t n_tok, int64_t n_seq, int64_t width,
                               nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_mingru_scan: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_seq >= 0 && n_seq <= 65535 && width > 0 && width < (1 << 30) && row_stride >= 3 * width && n_slots >= 0,
                NVX_EINVAL, "nvx_mingru_scan: bad sizes");
    if (n_tok == 0 || n_seq == 0) return NVX_OK;
    NVX_REQUIRE(zxg && state && pos0 && state_slot && out, NVX_EINVAL, "nvx_mingru_scan: null pointer");
    NVX_REQUIRE(qo_indptr || n_tok == n_seq, NVX_EINVAL, "nvx_mingru_scan: without qo_indptr every sequence has one token");
    NVX_FMT_DISPATCH(fmt, launch_mingru<A_>(zxg, row_stride, state, qo_indptr, pos0, state_slot, out, n_seq, (int)width, (hipStream_t)stream));
    return nvx_check_launch("nvx_mingru_scan");
}

extern "C" int nvx_rglru_scan(const void* y, int64_t y_stride, const void* u, int64_t u_stride, const void* gates, int64_t g_block_stride,
                              int64_t g_tok_stride, int64_t block_width, const float* gate_bias, const float* rate, int fmt, float* state,
                              int64_t n_slots, const int32_t* qo_indptr, const int64_t* pos0, const int32_t* state_slot, void* out,
                              int64_t n_tok, int64_t n_seq, int64_t width, nvx_stream_t stream) {
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, "nvx_rglru_scan: fmt must be 0, 1 or 2");
    NVX_REQUIRE(n_tok >= 0 && n_seq >= 0 && n_seq <= 65535 && width > 0 && width < (1 << 30) && n_slots >= 0 && block_width > 0 &&
                    width % block_width == 0 && y_stride >= width && u_stride >= width && g_tok_stride >= 2 * block_width && g_block_stride >= 0,
                NVX_EINVAL, "nvx_rglru_scan: bad sizes");
    if (n_tok == 0 || n_seq == 0) return NVX_OK;
    NVX_REQUIRE(y && u && gates && gate_bias && rate && state && pos0 && state_slot && out, NVX_EINVAL, "nvx_rglru_scan: null pointer");
    NVX_REQUIRE(qo_indptr || n_tok == n_seq, NVX_EINVAL, "nvx_rglru_scan: without qo_indptr every sequence has one token");
    const RglruIn in = {y, y_stride, u, u_stride, gates, g_block_stride, g_tok_stride, gate_bias, rate, (int)block_width, (int)width};
    NVX_FMT_DISPATCH(fmt, launch_rglru<A_>(in, state, qo_indptr, pos0, state_slot, out, n_seq, (hipStream_t)stream));
    return nvx_check_launch("nvx_rglru_scan");
}
