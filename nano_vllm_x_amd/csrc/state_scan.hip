// Token mixers that carry a matrix per head from token to token, and the small steps in front of them:
//   - short causal convolution over time per channel (optional bias, optional silu), its last inputs kept per sequence;
//   - token shift: every token's row mixed with its predecessor's by per-channel weights, the last row kept per sequence;
//   - three recurrences over a (key size x value size) memory per head:
//       mlstm   exponential input gate and sigmoid forget gate stabilised by a running maximum, normaliser vector;
//       delta   per-head decay, then a rank-one correction of the memory towards the new value along the key;
//       rwkv    per-key-channel decay, the current token read with a bonus before it is written;
//       decay   one constant decay per head, the token written before it is read (linear attention with a fixed decay).
// One kernel per recurrence serves prompts, portions of prompts and single decoded tokens: a workgroup takes one head of
// one sequence and a block of value columns, a thread keeps KR rows of one column in registers, P neighbouring lanes
// share a column and add their partial read-outs by lane exchange.  The tokens' keys, queries and values are staged
// through LDS TB tokens at a time (converted to float32, unit-normed where the design asks for it), so the sequential
// loop touches no global memory but its output.  Memory, normaliser, maximum, gates and decays are float32.
// A batch is ragged (see seq_mix.hip): qo_indptr / pos0 / state_slot; a sequence at position 0 takes zeros for its state.
#include "fmt_dev.h"

namespace NVX_NS {

// ---- short convolution (+ bias, + silu) ------------------------------------------------------------------------------------
// out[t][c] = act(bias[c] + sum_j w[j][c] * in[t - (taps_n - 1) + j][c]) over the tokens of t's own sequence (bias may be null; act 0:
// none, 1: silu); inputs before this step come from state[slot] (taps_n - 1 rows, oldest first), inputs before the sequence's
// start are zero.
template <typename A>
__global__ __launch_bounds__(256) void short_conv_kernel(const A* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                        const float* __restrict__ bias, int act, int taps_n, const float* __restrict__ state, const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                             const int32_t* __restrict__ state_slot, A* __restrict__ out, int channels) {
    const int64_t t = blockIdx.y;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const SeqSpan s = seq_span(b, qo_indptr, pos0, state_slot);
    const int64_t j = t - s.q0;
    const int hist_n = taps_n - 1;
    const bool has_state = s.pos0 > 0 && s.slot >= 0;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < channels; c += gridDim.x * 256) {
        float acc = bias ? bias[c] : 0.f;
        for (int i = 0; i < taps_n; ++i) {
            const int64_t src = j - (hist_n - i);
            float v = 0.f;
            if (src >= 0) v = ld_f(x, (s.q0 + src) * x_stride + c);
            else if (has_state) v = state[((int64_t)s.slot * hist_n + (hist_n + src)) * channels + c];
            acc += w[(int64_t)i * channels + c] * v;
        }
        st_f(out, t * (int64_t)channels + c, act == 1 ? acc * sigmoid_f(acc) : acc);
    }
}

// state[slot] <- the sequence's last hist_n inputs (older rows of the state move up where the step brought fewer).
template <typename A>
__global__ __launch_bounds__(256) void tail_rows_kernel(const A* __restrict__ x, int64_t x_stride, int hist_n, float* __restrict__ state,
                                                       const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                       const int32_t* __restrict__ state_slot, int channels) {
    const SeqSpan s = seq_span(blockIdx.y, qo_indptr, pos0, state_slot);
    if (s.slot < 0 || s.n <= 0) return;
    const bool has_state = s.pos0 > 0;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < channels; c += gridDim.x * 256) {
        float* st = state + (int64_t)s.slot * hist_n * channels + c;
        for (int r = 0; r < hist_n; ++r) {        // ascending: row r takes old row r + n, which is not yet overwritten
            const int64_t src = s.n - hist_n + r;
            float v;
            if (src >= 0) v = ld_f(x, (s.q0 + src) * x_stride + c);
            else v = has_state ? st[(int64_t)(r + s.n) * channels] : 0.f;
            st[(int64_t)r * channels] = v;
        }
    }
}

// out[m][t][c] = h[t][c] + (h[t-1][c] - h[t][c]) * mu[m][c]; the predecessor of a step's first token is state[slot].
template <typename A>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(const A* __restrict__ h, int64_t h_stride, const float* __restrict__ mu,
                                                             int n_mix, const float* __restrict__ state, const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                             const int32_t* __restrict__ state_slot, A* __restrict__ out, int64_t n_tok,
                                                             int width) {
    const int64_t t = blockIdx.y;
    const int b = tok_seq ? tok_seq[t] : (int)t;
    const SeqSpan s = seq_span(b, qo_indptr, pos0, state_slot);
    for (int c = blockIdx.x * 256 + threadIdx.x; c < width; c += gridDim.x * 256) {
        const float cur = ld_f(h, t * h_stride + c);
        float prev = 0.f;
        if (t > s.q0) prev = ld_f(h, (t - 1) * h_stride + c);
        else if (s.pos0 > 0 && s.slot >= 0) prev = state[(int64_t)s.slot * width + c];
        for (int m = 0; m < n_mix; ++m)
            st_f(out, ((int64_t)m * n_tok + t) * width + c, cur + (prev - cur) * mu[(int64_t)m * width + c]);
    }
}

// ---- matrix-memory recurrences ---------------------------------------------------------------------------------------------
constexpr int KR = 32;        // rows of a column that one thread keeps
constexpr int KS = KR + 4;    // LDS stride of such a group of rows (keeps 16-byte alignment, spreads the groups over banks)
constexpr int TB = 8;         // tokens staged at a time

__device__ __forceinline__ int lds_row(int d) { return (d / KR) * KS + (d % KR); }
__device__ __forceinline__ float lanes_sum(float v, int p_lanes) {
    for (int m = 1; m < p_lanes; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}

struct ScanThread { int col, p, e, r0; bool active; };
__device__ __forceinline__ ScanThread scan_thread(int p_lanes, int vdim) {
    ScanThread th;
    const int cb = blockDim.x / p_lanes;
    th.col = threadIdx.x / p_lanes;
    th.p = threadIdx.x % p_lanes;
    th.e = blockIdx.x * cb + th.col;
    th.r0 = th.p * KR;
    th.active = th.e < vdim;
    return th;
}

// stage `nt` tokens' rows of `dim` elements starting at column `off` of x into dst (row stride p_lanes * KS), times `mul`
template <typename A>
__device__ __forceinline__ void stage_rows(float* dst, const A* x, int64_t x_stride, int64_t tok0, int nt, int off, int dim, int p_lanes,
                                           float mul) {
    for (int i = threadIdx.x; i < nt * dim; i += blockDim.x) {
        const int tt = i / dim, d = i % dim;
        dst[tt * p_lanes * KS + lds_row(d)] = ld_f(x, (tok0 + tt) * x_stride + off + d) * mul;
    }
}
template <typename A>
__device__ __forceinline__ void stage_cols(float* dst, const A* x, int64_t x_stride, int64_t tok0, int nt, int off, int vdim, int cb) {
    for (int i = threadIdx.x; i < nt * cb; i += blockDim.x) {
        const int tt = i / cb, c = i % cb;
        const int e = blockIdx.x * cb + c;
        dst[i] = e < vdim ? ld_f(x, (tok0 + tt) * x_stride + off + e) : 0.f;
    }
}
__device__ __forceinline__ void zero_rows(float* dst, int n) {
    for (int i = threadIdx.x; i < n; i += blockDim.x) dst[i] = 0.f;
}
// rows of dst (nt of them, `dim` used elements each) scaled to unit length: x / sqrt(sum x^2 + 1e-6) * mul; a wave per row
__device__ __forceinline__ void unit_rows(float* dst, int nt, int dim, int p_lanes, float mul) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, n_waves = blockDim.x >> 6;
    for (int tt = wave; tt < nt; tt += n_waves) {
        float* r = dst + tt * p_lanes * KS;
        float ss = 0.f;
        for (int d = lane; d < dim; d += 64) { const float v = r[lds_row(d)]; ss += v * v; }
        const float sc = mul / sqrtf(wave_sum(ss) + 1e-6f);
        for (int d = lane; d < dim; d += 64) r[lds_row(d)] *= sc;
    }
}

// mLSTM.  x[t] holds q at q_off, k at k_off (heads * dim each) and v at v_off (heads * vdim); gates[t] = [i | f] pre-activations
// (heads each, float32), gate_bias likewise.  i = cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap));
//   m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;  o = S^T q / (max(|n.q|, e^(-m')) + 1e-6)
// with q scaled by dim^(-1/2); m starts at 0.  S: (slots, heads, dim, vdim), n: (slots, heads, dim), m: (slots, heads).
// Every column block of a head reads n and m (N_in, M_in) and the first one writes them (N, M): where a head has more than one
// column block the caller hands in copies to read from, since a block that starts late must not see the new values.
template <typename A>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(const A* __restrict__ x, int64_t x_stride, int q_off, int k_off, int v_off,
                                                        const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                                                        float* __restrict__ S, const float* __restrict__ N_in, const float* __restrict__ M_in,
                                                        float* __restrict__ N, float* __restrict__ M,
                                                        const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                        const int32_t* __restrict__ state_slot, float* __restrict__ out, int heads, int dim,
                                                        int vdim, int p_lanes) {
    extern __shared__ float sm[];
    const int cb = blockDim.x / p_lanes, rs = p_lanes * KS;
    float* sq = sm;
    float* sk = sq + TB * rs;
    float* sv = sk + TB * rs;
    float* si = sv + TB * cb;
    float* sf = si + TB;
    const int hd = blockIdx.y;
    const SeqSpan sp = seq_span(blockIdx.z, qo_indptr, pos0, state_slot);
    if (sp.slot < 0 || sp.n <= 0) return;
    const ScanThread th = scan_thread(p_lanes, vdim);
    float* Sp = S + ((int64_t)sp.slot * heads + hd) * dim * vdim;
    float* Np = N + ((int64_t)sp.slot * heads + hd) * dim;
    const float* Np_in = N_in + ((int64_t)sp.slot * heads + hd) * dim;
    float s[KR], nn[KR];
    float m = 0.f;
    const bool cont = sp.pos0 > 0;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        const bool in = cont && row < dim;
        s[r] = (in && th.active) ? Sp[(int64_t)row * vdim + th.e] : 0.f;
        nn[r] = in ? Np_in[row] : 0.f;
    }
    if (cont) m = M_in[(int64_t)sp.slot * heads + hd];
    zero_rows(sq, 2 * TB * rs);
    const float q_mul = 1.0f / sqrtf((float)dim);
    for (int64_t t0 = 0; t0 < sp.n; t0 += TB) {
        const int nt = (int)(sp.n - t0 < TB ? sp.n - t0 : TB);
        __syncthreads();
        stage_rows(sq, x, x_stride, sp.q0 + t0, nt, q_off + hd * dim, dim, p_lanes, q_mul);
        stage_rows(sk, x, x_stride, sp.q0 + t0, nt, k_off + hd * dim, dim, p_lanes, 1.0f);
        stage_cols(sv, x, x_stride, sp.q0 + t0, nt, v_off + hd * vdim, vdim, cb);
        if ((int)threadIdx.x < nt) {
            const float* g = gates + (sp.q0 + t0 + threadIdx.x) * 2 * heads;
            si[threadIdx.x] = cap * tanhf((g[hd] + gate_bias[hd]) / cap);
            sf[threadIdx.x] = logsigmoid_f(cap * tanhf((g[heads + hd] + gate_bias[heads + hd]) / cap));
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float gi = si[tt], gf = sf[tt];
            const float m_new = fmaxf(gf + m, gi);
            const float keep = expf(gf + m - m_new), put = expf(gi - m_new);
            m = m_new;
            const float v = sv[tt * cb + th.col];
            const float* kk = sk + tt * rs + th.p * KS;
            const float* qq = sq + tt * rs + th.p * KS;
            float num = 0.f, nq = 0.f;
#pragma unroll
            for (int r = 0; r < KR; ++r) {
                const float kp = put * kk[r];
                s[r] = keep * s[r] + kp * v;
                nn[r] = keep * nn[r] + kp;
                num += s[r] * qq[r];
                nq += nn[r] * qq[r];
            }
            num = lanes_sum(num, p_lanes);
            nq = lanes_sum(nq, p_lanes);
            if (th.p == 0 && th.active)
                out[(sp.q0 + t0 + tt) * (int64_t)heads * vdim + (int64_t)hd * vdim + th.e] = num / (fmaxf(fabsf(nq), expf(-m)) + 1e-6f);
        }
    }
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        if (row < dim && th.active) Sp[(int64_t)row * vdim + th.e] = s[r];
        if (row < dim && blockIdx.x == 0 && th.col == 0) Np[row] = nn[r];
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) M[(int64_t)sp.slot * heads + hd] = m;
}

// Gated delta rule.  x[t] holds q at q_off, k at k_off (kv_heads * dim each, after convolution and silu) and v at v_off (heads *
// vdim); ab[t] = [a | b] pre-activations (heads each, float32).  q and k are scaled to unit length per head (q also by
// dim^(-1/2)); g = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b);
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.          S: (slots, heads, dim, vdim).
template <typename A>
__global__ __launch_bounds__(256) void delta_scan_kernel(const A* __restrict__ x, int64_t x_stride, int q_off, int k_off, int v_off,
                                                        const float* __restrict__ ab, const float* __restrict__ a_log,
                                                        const float* __restrict__ dt_bias, float* __restrict__ S,
                                                        const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                        const int32_t* __restrict__ state_slot, float* __restrict__ out, int heads,
                                                        int kv_heads, int dim, int vdim, int p_lanes) {
    extern __shared__ float sm[];
    const int cb = blockDim.x / p_lanes, rs = p_lanes * KS;
    float* sq = sm;
    float* sk = sq + TB * rs;
    float* sv = sk + TB * rs;
    float* sg = sv + TB * cb;
    float* sb = sg + TB;
    const int hd = blockIdx.y, kvh = hd / (heads / kv_heads);
    const SeqSpan sp = seq_span(blockIdx.z, qo_indptr, pos0, state_slot);
    if (sp.slot < 0 || sp.n <= 0) return;
    const ScanThread th = scan_thread(p_lanes, vdim);
    float* Sp = S + ((int64_t)sp.slot * heads + hd) * dim * vdim;
    float s[KR];
    const bool cont = sp.pos0 > 0;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        s[r] = (cont && row < dim && th.active) ? Sp[(int64_t)row * vdim + th.e] : 0.f;
    }
    zero_rows(sq, 2 * TB * rs);
    const float rate = expf(a_log[hd]), bias = dt_bias[hd];
    const float q_mul = 1.0f / sqrtf((float)dim);
    for (int64_t t0 = 0; t0 < sp.n; t0 += TB) {
        const int nt = (int)(sp.n - t0 < TB ? sp.n - t0 : TB);
        __syncthreads();
        stage_rows(sq, x, x_stride, sp.q0 + t0, nt, q_off + kvh * dim, dim, p_lanes, 1.0f);
        stage_rows(sk, x, x_stride, sp.q0 + t0, nt, k_off + kvh * dim, dim, p_lanes, 1.0f);
        stage_cols(sv, x, x_stride, sp.q0 + t0, nt, v_off + hd * vdim, vdim, cb);
        if ((int)threadIdx.x < nt) {
            const float* g = ab + (sp.q0 + t0 + threadIdx.x) * 2 * heads;
            sg[threadIdx.x] = expf(-rate * softplus_f(g[hd] + bias));
            sb[threadIdx.x] = sigmoid_f(g[heads + hd]);
        }
        __syncthreads();
        unit_rows(sq, nt, dim, p_lanes, q_mul);
        unit_rows(sk, nt, dim, p_lanes, 1.0f);
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float g = sg[tt], beta = sb[tt];
            const float* kk = sk + tt * rs + th.p * KS;
            const float* qq = sq + tt * rs + th.p * KS;
            float kdot = 0.f;
#pragma unroll
            for (int r = 0; r < KR; ++r) {
                s[r] *= g;
                kdot += s[r] * kk[r];
            }
            kdot = lanes_sum(kdot, p_lanes);
            const float u = beta * (sv[tt * cb + th.col] - kdot);
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < KR; ++r) {
                s[r] += kk[r] * u;
                o += s[r] * qq[r];
            }
            o = lanes_sum(o, p_lanes);
            if (th.p == 0 && th.active) out[(sp.q0 + t0 + tt) * (int64_t)heads * vdim + (int64_t)hd * vdim + th.e] = o;
        }
    }
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        if (row < dim && th.active) Sp[(int64_t)row * vdim + th.e] = s[r];
    }
}

// RWKV-style time mixing.  r, k, v: (n_tok, heads * dim) each (rows rkv_stride apart); wlog (n_tok, heads * dim) float32 and w0
// (heads * dim): the decay of key channel c is w = exp(-exp(wlog + w0)); bonus (heads, dim).
//   o = (S + diag(bonus) k v^T)^T r;  S <- diag(w) S + k v^T.          S: (slots, heads, dim, dim).
template <typename A>
__global__ __launch_bounds__(256) void rwkv_scan_kernel(const A* __restrict__ rx, const A* __restrict__ kx, const A* __restrict__ vx,
                                                       int64_t rkv_stride, const float* __restrict__ wlog, const float* __restrict__ w0,
                                                       const float* __restrict__ bonus, float* __restrict__ S,
                                                       const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                       const int32_t* __restrict__ state_slot, float* __restrict__ out, int heads, int dim,
                                                       int p_lanes) {
    extern __shared__ float sm[];
    const int cb = blockDim.x / p_lanes, rs = p_lanes * KS;
    float* sr = sm;
    float* sk = sr + TB * rs;
    float* sw = sk + TB * rs;
    float* sv = sw + TB * rs;
    const int hd = blockIdx.y;
    const SeqSpan sp = seq_span(blockIdx.z, qo_indptr, pos0, state_slot);
    if (sp.slot < 0 || sp.n <= 0) return;
    const ScanThread th = scan_thread(p_lanes, dim);
    float* Sp = S + ((int64_t)sp.slot * heads + hd) * dim * dim;
    float s[KR], uu[KR];
    const bool cont = sp.pos0 > 0;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        s[r] = (cont && row < dim && th.active) ? Sp[(int64_t)row * dim + th.e] : 0.f;
        uu[r] = row < dim ? bonus[hd * dim + row] : 0.f;
    }
    zero_rows(sr, 3 * TB * rs);
    for (int64_t t0 = 0; t0 < sp.n; t0 += TB) {
        const int nt = (int)(sp.n - t0 < TB ? sp.n - t0 : TB);
        __syncthreads();
        stage_rows(sr, rx, rkv_stride, sp.q0 + t0, nt, hd * dim, dim, p_lanes, 1.0f);
        stage_rows(sk, kx, rkv_stride, sp.q0 + t0, nt, hd * dim, dim, p_lanes, 1.0f);
        stage_cols(sv, vx, rkv_stride, sp.q0 + t0, nt, hd * dim, dim, cb);
        for (int i = threadIdx.x; i < nt * dim; i += blockDim.x) {
            const int tt = i / dim, d = i % dim;
            sw[tt * rs + lds_row(d)] = expf(-expf(wlog[(sp.q0 + t0 + tt) * (int64_t)heads * dim + hd * dim + d] + w0[hd * dim + d]));
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float v = sv[tt * cb + th.col];
            const float* rr = sr + tt * rs + th.p * KS;
            const float* kk = sk + tt * rs + th.p * KS;
            const float* ww = sw + tt * rs + th.p * KS;
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < KR; ++r) {
                const float kv = kk[r] * v;
                o += rr[r] * (s[r] + uu[r] * kv);
                s[r] = ww[r] * s[r] + kv;
            }
            o = lanes_sum(o, p_lanes);
            if (th.p == 0 && th.active) out[(sp.q0 + t0 + tt) * (int64_t)heads * dim + (int64_t)hd * dim + th.e] = o;
        }
    }
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        if (row < dim && th.active) Sp[(int64_t)row * dim + th.e] = s[r];
    }
}

// Linear attention with a constant decay per head.  x[t] holds q at q_off, k at k_off (heads * dim each) and v at v_off (heads *
// vdim), pre-activations if act == 1 (silu is applied to all three as they are staged), values as they are if act == 0.
//   S <- decay[h] S + k v^T;  o = S^T q  (the read sees the token's own write).          S: (slots, heads, dim, vdim).
// Long portions are cut into chunks of `chunk` tokens that run side by side (blockIdx.z = sequence * n_chunk_max + chunk), in three
// launches: phase 1 builds every chunk's own contribution from a zero state into ws (no read-out), the carry kernel turns ws into
// the state at every chunk's start (and writes the sequence's final state), phase 3 walks every chunk from there with the read-out.
// Because the decay is a constant, the carry over a chunk of n tokens is decay^n S + (the chunk's own contribution).  phase 0: one
// workgroup walks the whole portion (single tokens, short portions).
__device__ __forceinline__ float scan_act(float z, int act) { return act == 1 ? z * sigmoid_f(z) : z; }
// `tb` tokens are staged at a time: 32 where the key size leaves LDS for them (more than the other recurrences take: an activation
// is applied as they are staged, and fewer, longer stages hide more of the loads), fewer for wide keys.
template <typename A, int PHASE>
__global__ __launch_bounds__(256) void decay_scan_kernel(const A* __restrict__ x, int64_t x_stride, int q_off, int k_off, int v_off, int act,
                                                        const float* __restrict__ decay, float* __restrict__ S,
                                                        const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                        const int32_t* __restrict__ state_slot, float* __restrict__ out, int heads, int dim,
                                                        int vdim, int p_lanes, int tb, int chunk, int n_chunk_max, float* __restrict__ ws) {
    constexpr int phase = PHASE;
    extern __shared__ float sm[];
    const int cb = blockDim.x / p_lanes, rs = p_lanes * KS;
    float* sq = sm;
    float* sk = sq + tb * rs;
    float* sv = sk + tb * rs;
    const int hd = blockIdx.y;
    const int seq = phase ? blockIdx.z / n_chunk_max : blockIdx.z, ck = phase ? blockIdx.z % n_chunk_max : 0;
    SeqSpan sp = seq_span(seq, qo_indptr, pos0, state_slot);
    if (sp.slot < 0 || sp.n <= 0) return;
    if (phase) {                                     // this workgroup's chunk of the portion
        const int64_t first = (int64_t)ck * chunk;
        if (first >= sp.n) return;
        sp.q0 += first;
        sp.n = sp.n - first < chunk ? sp.n - first : chunk;
    }
    const ScanThread th = scan_thread(p_lanes, vdim);
    // where the state comes from and goes to: the pool (phase 0), nothing and ws (1), ws and nothing (3)
    float* Sp = phase ? ws + ((int64_t)blockIdx.z * heads + hd) * dim * vdim : S + ((int64_t)sp.slot * heads + hd) * dim * vdim;
    float s[KR];
    const bool cont = phase == 3 || (phase == 0 && sp.pos0 > 0);
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        s[r] = (cont && row < dim && th.active) ? Sp[(int64_t)row * vdim + th.e] : 0.f;
    }
    zero_rows(sq, 2 * tb * rs);
    const float g = decay[hd];
    for (int64_t t0 = 0; t0 < sp.n; t0 += tb) {
        const int nt = (int)(sp.n - t0 < tb ? sp.n - t0 : tb);
        __syncthreads();
        for (int i = threadIdx.x; i < nt * dim; i += blockDim.x) {
            const int tt = i / dim, d = i % dim;
            const int64_t r = (sp.q0 + t0 + tt) * x_stride + hd * dim + d;
            if (phase != 1) sq[tt * rs + lds_row(d)] = scan_act(ld_f(x, r + q_off), act);      // (phase 1 wants the state only)
            sk[tt * rs + lds_row(d)] = scan_act(ld_f(x, r + k_off), act);
        }
        for (int i = threadIdx.x; i < nt * cb; i += blockDim.x) {
            const int tt = i / cb, c = i % cb;
            const int e = blockIdx.x * cb + c;
            sv[i] = e < vdim ? scan_act(ld_f(x, (sp.q0 + t0 + tt) * x_stride + v_off + hd * vdim + e), act) : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float v = sv[tt * cb + th.col];
            const float* kk = sk + tt * rs + th.p * KS;
            const float* qq = sq + tt * rs + th.p * KS;
            if (phase == 1) {
#pragma unroll
                for (int r = 0; r < KR; ++r) s[r] = g * s[r] + kk[r] * v;
                continue;
            }
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < KR; ++r) {
                s[r] = g * s[r] + kk[r] * v;
                o += s[r] * qq[r];
            }
            o = lanes_sum(o, p_lanes);
            if (th.p == 0 && th.active) out[(sp.q0 + t0 + tt) * (int64_t)heads * vdim + (int64_t)hd * vdim + th.e] = o;
        }
    }
    if (phase == 3) return;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
        const int row = th.r0 + r;
        if (row < dim && th.active) Sp[(int64_t)row * vdim + th.e] = s[r];
    }
}

// Between the two chunked phases: ws[sequence][chunk] holds every chunk's own contribution and is replaced by the state at the chunk's
// start; the state after the last chunk goes to the pool.  One thread per element of a sequence's state.
__global__ __launch_bounds__(256) void decay_chunk_carry_kernel(const float* __restrict__ decay, float* __restrict__ S, float* __restrict__ ws,
                                                               const int32_t* __restrict__ qo_indptr, const int64_t* __restrict__ pos0,
                                                               const int32_t* __restrict__ state_slot, int heads, int dim, int vdim, int chunk,
                                                               int n_chunk_max) {
    const SeqSpan sp = seq_span(blockIdx.y, qo_indptr, pos0, state_slot);
    if (sp.slot < 0 || sp.n <= 0) return;
    const int64_t per = (int64_t)heads * dim * vdim;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= per) return;
    const float g = decay[i / ((int64_t)dim * vdim)];
    float* Sp = S + (int64_t)sp.slot * per + i;
    float run = sp.pos0 > 0 ? *Sp : 0.f;
    for (int ck = 0; (int64_t)ck * chunk < sp.n; ++ck) {
        const int64_t n = sp.n - (int64_t)ck * chunk < chunk ? sp.n - (int64_t)ck * chunk : chunk;
        float* w = ws + ((int64_t)blockIdx.y * n_chunk_max + ck) * per + i;
        const float own = *w;
        *w = run;
        float gn = 1.f;
        for (int64_t k = 0; k < n; ++k) gn *= g;     // the same products, in the same order, as n steps of the recurrence
        run = gn * run + own;
    }
    *Sp = run;
}

// launch geometry of the three recurrences: lanes per column (a power of two), threads per workgroup, value columns per
// workgroup
struct ScanLaunch { int p_lanes, threads, cb; };
static bool scan_launch(int64_t dim, int64_t vdim, ScanLaunch* g) {
    int p = 1;
    while ((int64_t)p * KR < dim) p <<= 1;
    if (p > 16) return false;                       // dim <= 512: two staged operands of TB tokens fit the default LDS window
    int64_t threads = ((vdim * p + 63) / 64) * 64;
    if (threads > 256) threads = 256;
    g->p_lanes = p;
    g->threads = (int)threads;
    g->cb = (int)threads / p;
    return true;
}

}  // namespace NVX_NS

using namespace NVX_NS;

#define NVX_LAYOUT_OK(name)                                                                                                         \
    NVX_REQUIRE(fmt >= 0 && fmt <= 2, NVX_EINVAL, name ": fmt must be 0, 1 or 2");                                                  \
    NVX_REQUIRE(n_tok >= 0 && n_seq >= 0 && n_seq <= 65535 && n_tok <= 65535 * 256, NVX_EINVAL, name ": bad token or sequence count"); \
    if (n_tok == 0 || n_seq == 0) return NVX_OK;                                                                                    \
    NVX_REQUIRE(pos0 && state_slot, NVX_EINVAL, name ": null layout");                                                              \
    NVX_REQUIRE(qo_indptr || n_tok == n_seq, NVX_EINVAL, name ": without qo_indptr every sequence has one token")

extern "C" int nvx_short_conv(const void* x, int64_t x_stride, int fmt, const float* w, const float* bias, int act, int taps_n, float* state,
                              int64_t n_slots, const int32_t* tok_seq, const int32_t* qo_indptr, const int64_t* pos0,
                              const int32_t* state_slot, void* out, int64_t n_tok, int64_t n_seq, int64_t channels, nvx_stream_t stream) {
    NVX_LAYOUT_OK("nvx_short_conv");
    NVX_REQUIRE(channels > 0 && channels < (1 << 30) && x_stride >= channels && taps_n >= 1 && taps_n <= 64 && n_slots >= 0 && n_tok <= 65535 &&
                    (act == 0 || act == 1), NVX_EINVAL, "nvx_short_conv: bad sizes, or an activation other than 0 (none) and 1 (silu)");
    NVX_REQUIRE(x && w && out && (state || taps_n == 1), NVX_EINVAL, "nvx_short_conv: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_short_conv: tok_seq and qo_indptr go together");
    const unsigned cx = (unsigned)((channels + 255) / 256);
    NVX_FMT_CALL(fmt, {
        hipLaunchKernelGGL(short_conv_kernel<A_>, dim3(cx, (unsigned)n_tok), dim3(256), 0, (hipStream_t)stream, (const A_*)x, x_stride, w, bias,
                           act, taps_n, (const float*)state, tok_seq, qo_indptr, pos0, state_slot, (A_*)out, (int)channels);
        if (taps_n > 1)
            hipLaunchKernelGGL(tail_rows_kernel<A_>, dim3(cx, (unsigned)n_seq), dim3(256), 0, (hipStream_t)stream, (const A_*)x, x_stride,
                               taps_n - 1, state, qo_indptr, pos0, state_slot, (int)channels);
    });
    return nvx_check_launch("nvx_short_conv");
}

extern "C" int nvx_short_conv_silu(const void* x, int64_t x_stride, int fmt, const float* w, int taps_n, float* state, int64_t n_slots,
                                   const int32_t* tok_seq, const int32_t* qo_indptr, const int64_t* pos0, const int32_t* state_slot,
                                   void* out, int64_t n_tok, int64_t n_seq, int64_t channels, nvx_stream_t stream) {
    return nvx_short_conv(x, x_stride, fmt, w, nullptr, 1, taps_n, state, n_slots, tok_seq, qo_indptr, pos0, state_slot, out, n_tok, n_seq,
                          channels, stream);
}

extern "C" int nvx_token_shift_mix(const void* h, int64_t h_stride, int fmt, const float* mu, int n_mix, float* state, int64_t n_slots,
                                   const int32_t* tok_seq, const int32_t* qo_indptr, const int64_t* pos0, const int32_t* state_slot,
                                   void* out, int64_t n_tok, int64_t n_seq, int64_t width, nvx_stream_t stream) {
    NVX_LAYOUT_OK("nvx_token_shift_mix");
    NVX_REQUIRE(width > 0 && width < (1 << 30) && h_stride >= width && n_mix >= 1 && n_mix <= 64 && n_slots >= 0 && n_tok <= 65535, NVX_EINVAL,
                "nvx_token_shift_mix: bad sizes");
    NVX_REQUIRE(h && mu && out && state, NVX_EINVAL, "nvx_token_shift_mix: null pointer");
    NVX_REQUIRE((tok_seq != nullptr) == (qo_indptr != nullptr), NVX_EINVAL, "nvx_token_shift_mix: tok_seq and qo_indptr go together");
    const unsigned cx = (unsigned)((width + 255) / 256);
    NVX_FMT_CALL(fmt, {
        hipLaunchKernelGGL(token_shift_mix_kernel<A_>, dim3(cx, (unsigned)n_tok), dim3(256), 0, (hipStream_t)stream, (const A_*)h, h_stride, mu,
                           n_mix, (const float*)state, tok_seq, qo_indptr, pos0, state_slot, (A_*)out, n_tok, (int)width);
        hipLaunchKernelGGL(tail_rows_kernel<A_>, dim3(cx, (unsigned)n_seq), dim3(256), 0, (hipStream_t)stream, (const A_*)h, h_stride, 1, state,
                           qo_indptr, pos0, state_slot, (int)width);
    });
    return nvx_check_launch("nvx_token_shift_mix");
}

extern "C" int64_t nvx_scan_column_blocks(int64_t dim, int64_t vdim) {
    ScanLaunch g;
    if (dim <= 0 || vdim <= 0 || !scan_launch(dim, vdim, &g)) return 0;
    return (vdim + g.cb - 1) / g.cb;
}

extern "C" int nvx_mlstm_scan(const void* x, int64_t x_stride, int fmt, int64_t q_off, int64_t k_off, int64_t v_off, const float* gates,
                              const float* gate_bias, float cap, float* S, const float* N_in, const float* M_in, float* N, float* M,
                              int64_t n_slots, const int32_t* qo_indptr,
                              const int64_t* pos0, const int32_t* state_slot, float* out, int64_t n_tok, int64_t n_seq, int64_t heads,
                              int64_t dim, int64_t vdim, nvx_stream_t stream) {
    NVX_LAYOUT_OK("nvx_mlstm_scan");
    ScanLaunch g;
    NVX_REQUIRE(heads > 0 && heads <= 65535 && dim > 0 && vdim > 0 && vdim < (1 << 24) && n_slots >= 0 && cap > 0.f, NVX_EINVAL,
                "nvx_mlstm_scan: bad sizes");
    NVX_REQUIRE(scan_launch(dim, vdim, &g), NVX_EUNSUPPORTED, "nvx_mlstm_scan: key size above 512");
    NVX_REQUIRE(x && gates && gate_bias && S && N && M && N_in && M_in && out, NVX_EINVAL, "nvx_mlstm_scan: null pointer");
    NVX_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && x_stride >= q_off + heads * dim && x_stride >= k_off + heads * dim &&
                    x_stride >= v_off + heads * vdim, NVX_EINVAL, "nvx_mlstm_scan: q, k or v lies outside a row");
    const size_t lds = (size_t)(2 * TB * g.p_lanes * KS + TB * g.cb + 2 * TB) * sizeof(float);
    const dim3 grid((unsigned)((vdim + g.cb - 1) / g.cb), (unsigned)heads, (unsigned)n_seq);
    NVX_REQUIRE(grid.x == 1 || (N_in != N && M_in != M), NVX_EINVAL,
                "nvx_mlstm_scan: a head with several column blocks reads its normaliser and maximum from copies");
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(mlstm_scan_kernel<A_>, grid, dim3(g.threads), lds, (hipStream_t)stream, (const A_*)x, x_stride, (int)q_off,
                                         (int)k_off, (int)v_off, gates, gate_bias, cap, S, N_in, M_in, N, M, qo_indptr, pos0, state_slot, out, (int)heads,
                                         (int)dim, (int)vdim, g.p_lanes));
    return nvx_check_launch("nvx_mlstm_scan");
}

extern "C" int nvx_delta_scan(const void* x, int64_t x_stride, int fmt, int64_t q_off, int64_t k_off, int64_t v_off, const float* ab,
                              const float* a_log, const float* dt_bias, float* S, int64_t n_slots, const int32_t* qo_indptr,
                              const int64_t* pos0, const int32_t* state_slot, float* out, int64_t n_tok, int64_t n_seq, int64_t heads,
                              int64_t kv_heads, int64_t dim, int64_t vdim, nvx_stream_t stream) {
    NVX_LAYOUT_OK("nvx_delta_scan");
    ScanLaunch g;
    NVX_REQUIRE(heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && vdim < (1 << 24) && n_slots >= 0,
                NVX_EINVAL, "nvx_delta_scan: bad sizes");
    NVX_REQUIRE(scan_launch(dim, vdim, &g), NVX_EUNSUPPORTED, "nvx_delta_scan: key size above 512");
    NVX_REQUIRE(x && ab && a_log && dt_bias && S && out, NVX_EINVAL, "nvx_delta_scan: null pointer");
    NVX_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && x_stride >= q_off + kv_heads * dim && x_stride >= k_off + kv_heads * dim &&
                    x_stride >= v_off + heads * vdim, NVX_EINVAL, "nvx_delta_scan: q, k or v lies outside a row");
    const size_t lds = (size_t)(2 * TB * g.p_lanes * KS + TB * g.cb + 2 * TB) * sizeof(float);
    const dim3 grid((unsigned)((vdim + g.cb - 1) / g.cb), (unsigned)heads, (unsigned)n_seq);
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(delta_scan_kernel<A_>, grid, dim3(g.threads), lds, (hipStream_t)stream, (const A_*)x, x_stride, (int)q_off,
                                         (int)k_off, (int)v_off, ab, a_log, dt_bias, S, qo_indptr, pos0, state_slot, out, (int)heads,
                                         (int)kv_heads, (int)dim, (int)vdim, g.p_lanes));
    return nvx_check_launch("nvx_delta_scan");
}

extern "C" int nvx_rwkv_scan(const void* r, const void* k, const void* v, int64_t rkv_stride, int fmt, const float* wlog, const float* w0,
                             const float* bonus, float* S, int64_t n_slots, const int32_t* qo_indptr, const int64_t* pos0,
                             const int32_t* state_slot, float* out, int64_t n_tok, int64_t n_seq, int64_t heads, int64_t dim,
                             nvx_stream_t stream) {
    NVX_LAYOUT_OK("nvx_rwkv_scan");
    ScanLaunch g;
    NVX_REQUIRE(heads > 0 && heads <= 65535 && dim > 0 && n_slots >= 0 && rkv_stride >= heads * dim, NVX_EINVAL, "nvx_rwkv_scan: bad sizes");
    NVX_REQUIRE(scan_launch(dim, dim, &g) && g.p_lanes <= 8, NVX_EUNSUPPORTED, "nvx_rwkv_scan: head size above 256");
    NVX_REQUIRE(r && k && v && wlog && w0 && bonus && S && out, NVX_EINVAL, "nvx_rwkv_scan: null pointer");
    const size_t lds = (size_t)(3 * TB * g.p_lanes * KS + TB * g.cb) * sizeof(float);
    const dim3 grid((unsigned)((dim + g.cb - 1) / g.cb), (unsigned)heads, (unsigned)n_seq);
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL(rwkv_scan_kernel<A_>, grid, dim3(g.threads), lds, (hipStream_t)stream, (const A_*)r, (const A_*)k,
                                         (const A_*)v, rkv_stride, wlog, w0, bonus, S, qo_indptr, pos0, state_slot, out, (int)heads, (int)dim,
                                         g.p_lanes));
    return nvx_check_launch("nvx_rwkv_scan");
}

extern "C" int nvx_decay_scan(const void* x, int64_t x_stride, int fmt, int64_t q_off, int64_t k_off, int64_t v_off, int act,
                              const float* decay, float* S, int64_t n_slots, const int32_t* qo_indptr, const int64_t* pos0,
                              const int32_t* state_slot, float* out, int64_t n_tok, int64_t n_seq, int64_t heads, int64_t dim, int64_t vdim,
                              int64_t chunk, int64_t n_chunk_max, float* ws, nvx_stream_t stream) {
    NVX_LAYOUT_OK("nvx_decay_scan");
    ScanLaunch g;
    NVX_REQUIRE(heads > 0 && heads <= 65535 && dim > 0 && vdim > 0 && vdim < (1 << 24) && n_slots >= 0 && (act == 0 || act == 1), NVX_EINVAL,
                "nvx_decay_scan: bad sizes");
    NVX_REQUIRE(scan_launch(dim, vdim, &g), NVX_EUNSUPPORTED, "nvx_decay_scan: key size above 512");
    NVX_REQUIRE(x && decay && S && out, NVX_EINVAL, "nvx_decay_scan: null pointer");
    NVX_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && x_stride >= q_off + heads * dim && x_stride >= k_off + heads * dim &&
                    x_stride >= v_off + heads * vdim, NVX_EINVAL, "nvx_decay_scan: q, k or v lies outside a row");
    const int tb = g.p_lanes <= 4 ? 32 : (g.p_lanes == 8 ? 16 : TB);
    const size_t lds = (size_t)(2 * tb * g.p_lanes * KS + tb * g.cb) * sizeof(float);
    NVX_REQUIRE(chunk == 0 || (chunk > 0 && chunk < (1 << 30) && n_chunk_max > 0 && n_seq * n_chunk_max <= 65535 && ws && qo_indptr), NVX_EINVAL,
                "nvx_decay_scan: chunks need a ragged step, their workspace, and at most 65535 of them");
    const dim3 grid((unsigned)((vdim + g.cb - 1) / g.cb), (unsigned)heads, (unsigned)(chunk ? n_seq * n_chunk_max : n_seq));
#define NVX_DECAY_SCAN(PHASE)                                                                                                                      \
    NVX_FMT_CALL(fmt, hipLaunchKernelGGL((decay_scan_kernel<A_, PHASE>), grid, dim3(g.threads), lds, (hipStream_t)stream, (const A_*)x, x_stride,   \
                                         (int)q_off, (int)k_off, (int)v_off, act, decay, S, qo_indptr, pos0, state_slot, out, (int)heads, (int)dim,  \
                                         (int)vdim, g.p_lanes, tb, (int)chunk, (int)n_chunk_max, ws))
    if (!chunk) {
        NVX_DECAY_SCAN(0);
    } else {
        NVX_DECAY_SCAN(1);
        hipLaunchKernelGGL(decay_chunk_carry_kernel, dim3((unsigned)((heads * dim * vdim + 255) / 256), (unsigned)n_seq), dim3(256), 0,
                           (hipStream_t)stream, decay, S, ws, qo_indptr, pos0, state_slot, (int)heads, (int)dim, (int)vdim, (int)chunk,
                           (int)n_chunk_max);
        NVX_DECAY_SCAN(3);
    }
#undef NVX_DECAY_SCAN
    return nvx_check_launch("nvx_decay_scan");
}
