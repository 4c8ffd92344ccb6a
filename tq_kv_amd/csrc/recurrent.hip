// Mixers that carry a fixed-size state from token to token instead of keys and values: a short causal convolution per
// channel whose first inputs come from the state, the gated linear recurrence of a real-gated linear recurrent unit
// (RG-LRU), and the selective state-space recurrence with a scalar decay per head (the Mamba-2 form).  Everything that
// enters a recurrence is float32: decays, step sizes, gates, the state itself.  A step is a packed batch: token t belongs
// to sequence tok_seq[t] of the step, sequence s brings seq_new[s] tokens from packed row cu[s] on, and its state is row
// seq_slot[s] of the state tensor (rows state_stride floats apart).  All sizes a launch depends on are the step's shape;
// positions, slots and counts are read on the device, so a step of one token a sequence replays from a graph.
//
//   conv:    u_t[c] = bias[c] + sum_k w[c][k] x_(t - (taps-1-k))[c]        (inputs before the sequence's start are zero)
//   rg-lru:  r = sigmoid(Wa u + ba), i = sigmoid(Wi u + bi) block by block;  log a = c r with c = -8 softplus(lam)
//            S_t = a S_(t-1) + sqrt(1 - a^2) i u;  out_t = S_t gelu_tanh(y_t)
//   ssm:     dt = softplus(dt_raw + dt_bias);  S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T;  y_t = S_t^T C_t + D x_t
//   gated norm: v = y silu(z);  out = v / rms(v over its part) * w
#include "common.h"
#include "tq_kernels.h"

__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }
__device__ __forceinline__ float sigmoid_f(float v) { return 1.f / (1.f + expf(-v)); }
__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float gelu_tanh_f(float g) { return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))); }

// ---- the convolution ----------------------------------------------------------------------------------
// A thread per (token, channel).  state holds the sequence's last taps - 1 inputs, oldest first, [taps - 1][channels].
template <typename TA>
__global__ __launch_bounds__(256)
void conv_state_kernel(const TA* __restrict__ x, long long x_stride, const float* __restrict__ in_bias, const float* __restrict__ w,
                       const float* __restrict__ bias, int taps, int activation, const float* __restrict__ state, long long state_stride,
                       const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ seq_slot,
                       const int32_t* __restrict__ seq_start, float* __restrict__ out, int channels) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int seq = tok_seq[t];
    const int j = tok_pos[t] - seq_start[seq];           // the token's place among those the step brings of its sequence
    const float* st = state + (size_t)seq_slot[seq] * state_stride;
    const float ib = in_bias ? in_bias[c] : 0.f;
    float acc = 0.f;
    for (int k = 0; k < taps; ++k) {
        const int back = taps - 1 - k;
        float v;
        if (j - back >= 0) v = to_float(x[(size_t)(t - back) * x_stride + c]) + ib;
        else v = st[(size_t)(taps - 1 + j - back) * channels + c];
        acc = fmaf(w[(size_t)c * taps + k], v, acc);
    }
    acc += bias ? bias[c] : 0.f;
    if (activation == 1) acc = silu_f(acc);
    out[(size_t)t * channels + c] = acc;
}

// Four values of a row at an aligned place
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
    const float4 f = *reinterpret_cast<const float4*>(p);
    v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&v)[4]) {
    const uint2 h = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(h.x << 16); v[1] = __uint_as_float(h.x & 0xffff0000u);
    v[2] = __uint_as_float(h.y << 16); v[3] = __uint_as_float(h.y & 0xffff0000u);
}

// The same for steps of many rows: a thread takes four neighbouring channels of CONV_ROWS consecutive rows, reads every
// input once (the rows' window of CONV_ROWS + TAPS - 1 inputs stays in registers) and the four channels together.  A tap
// that reaches back before the step's first token of its sequence reads the state instead, as above, and the sum over
// the taps runs in the same order.
#define CONV_ROWS 8
template <typename TA, int TAPS>
__global__ __launch_bounds__(128)
void conv_state_vec_kernel(const TA* __restrict__ x, long long x_stride, const float* __restrict__ in_bias, const float* __restrict__ w,
                           const float* __restrict__ bias, int activation, const float* __restrict__ state, long long state_stride,
                           const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ seq_slot,
                           const int32_t* __restrict__ seq_start, float* __restrict__ out, int n_tokens, int channels) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c >= channels) return;
    const int t0 = blockIdx.y * CONV_ROWS;
    float wv[4][TAPS], ib[4], bv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int k = 0; k < TAPS; ++k) wv[j][k] = w[(size_t)(c + j) * TAPS + k];
        ib[j] = in_bias ? in_bias[c + j] : 0.f;
        bv[j] = bias ? bias[c + j] : 0.f;
    }
    float in[CONV_ROWS + TAPS - 1][4];
#pragma unroll
    for (int r = 0; r < CONV_ROWS + TAPS - 1; ++r) {
        const int t = t0 + r - (TAPS - 1);
        if (t >= 0 && t < n_tokens) {
            load4(x + (size_t)t * x_stride + c, in[r]);
#pragma unroll
            for (int j = 0; j < 4; ++j) in[r][j] += ib[j];
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) in[r][j] = 0.f;
        }
    }
#pragma unroll
    for (int r = 0; r < CONV_ROWS; ++r) {
        const int t = t0 + r;
        if (t < n_tokens) {
            const int seq = tok_seq[t];
            const int jpos = tok_pos[t] - seq_start[seq];
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            if (jpos >= TAPS - 1) {
#pragma unroll
                for (int k = 0; k < TAPS; ++k)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[j] = fmaf(wv[j][k], in[r + k][j], acc[j]);
            } else {
                const float* st = state + (size_t)seq_slot[seq] * state_stride + c;
#pragma unroll
                for (int k = 0; k < TAPS; ++k) {
                    const int back = TAPS - 1 - k;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float v = jpos - back >= 0 ? in[r + k][j] : st[(size_t)(TAPS - 1 + jpos - back) * channels + j];
                        acc[j] = fmaf(wv[j][k], v, acc[j]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] += bv[j];
                if (activation == 1) acc[j] = silu_f(acc[j]);
            }
            *reinterpret_cast<float4*>(out + (size_t)t * channels + c) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        }
    }
}

// The state after the step: the last taps - 1 inputs of each sequence, from the step's rows or, where the step brought
// fewer, from the state before.  A thread per (sequence, channel) reads all it needs before it writes.
template <typename TA>
__global__ __launch_bounds__(256)
void conv_state_update_kernel(const TA* __restrict__ x, long long x_stride, const float* __restrict__ in_bias, int taps, float* __restrict__ state,
                              long long state_stride, const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_new,
                              const int32_t* __restrict__ seq_slot, int channels) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int n = seq_new[s], keep = taps - 1;
    if (n <= 0) return;
    float* st = state + (size_t)seq_slot[s] * state_stride;
    const float ib = in_bias ? in_bias[c] : 0.f;
    float held[TQK_CONV_MAX_TAPS - 1];
#pragma unroll
    for (int i = 0; i < TQK_CONV_MAX_TAPS - 1; ++i) {
        if (i >= keep) break;
        const int from_end = keep - i;                // this entry is the input `from_end` tokens before the step's end
        if (from_end <= n) held[i] = to_float(x[(size_t)(cu[s] + n - from_end) * x_stride + c]) + ib;
        else held[i] = st[(size_t)(i + n) * channels + c];
    }
#pragma unroll
    for (int i = 0; i < TQK_CONV_MAX_TAPS - 1; ++i) {
        if (i >= keep) break;
        st[(size_t)i * channels + c] = held[i];
    }
}

// Steps of one token a sequence: output and new state in one launch.  A thread per (token, channel) reads the state's
// taps - 1 inputs, sums in the order of the kernels above, and writes the state moved on by its token's input.
template <typename TA>
__global__ __launch_bounds__(256)
void conv_state_step_kernel(const TA* __restrict__ x, long long x_stride, const float* __restrict__ in_bias, const float* __restrict__ w,
                            const float* __restrict__ bias, int taps, int activation, float* __restrict__ state, long long state_stride,
                            const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ seq_slot, float* __restrict__ out, int channels) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    float* st = state + (size_t)seq_slot[tok_seq[t]] * state_stride + c;
    const float v_new = to_float(x[(size_t)t * x_stride + c]) + (in_bias ? in_bias[c] : 0.f);
    const int keep = taps - 1;
    float held[TQK_CONV_MAX_TAPS - 1];
#pragma unroll
    for (int i = 0; i < TQK_CONV_MAX_TAPS - 1; ++i) held[i] = i < keep ? st[(size_t)i * channels] : 0.f;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < TQK_CONV_MAX_TAPS - 1; ++i)
        if (i < keep) acc = fmaf(w[(size_t)c * taps + i], held[i], acc);
    acc = fmaf(w[(size_t)c * taps + keep], v_new, acc);
    acc += bias ? bias[c] : 0.f;
    if (activation == 1) acc = silu_f(acc);
    out[(size_t)t * channels + c] = acc;
#pragma unroll
    for (int i = 0; i < TQK_CONV_MAX_TAPS - 1; ++i)
        if (i < keep) st[(size_t)i * channels] = i + 1 < keep ? held[i + 1 < TQK_CONV_MAX_TAPS - 1 ? i + 1 : i] : v_new;
}

// ---- gates of the RG-LRU ---------------------------------------------------------------------------------
// The two gates' matrices are block-diagonal: `blocks` square matrices of bs = width / blocks.  wa_t and wi_t hold them
// with the input index first, [blocks][bs in][bs out], so that neighbouring threads read neighbouring outputs.  A block
// of threads takes RG_TOKENS tokens and one diagonal block; the tokens' inputs wait in LDS, [bs][RG_TOKENS], so that a
// thread reads an input of all the tokens in two pieces of 16 bytes.
// KS = 1: a thread per output, up to 256 of them a block; the sum over the inputs runs in their order, whatever else the
// step holds.  KS = RG_TOKENS: steps of few tokens, where that would leave a few waves walking all the inputs one after
// the other: a block takes 256 / KS outputs, the inputs are dealt out to KS slices of threads, the slices' sums meet in
// LDS, and slice k finishes token k.
#define RG_TOKENS 8
template <int KS>
__global__ __launch_bounds__(256)
void rglru_gates_kernel(const float* __restrict__ u, const float* __restrict__ wa_t, const float* __restrict__ wi_t, const float* __restrict__ ba,
                        const float* __restrict__ bi, const float* __restrict__ decay_c, float* __restrict__ a_out, float* __restrict__ g_out,
                        int n_tokens, int width, int bs) {
    static_assert(KS == 1 || KS == RG_TOKENS, "a slice finishes a token");
    extern __shared__ __align__(16) float u_lds[];    // [bs][RG_TOKENS], then (KS > 1) the slices' sums [KS][2][RG_TOKENS][outputs]
    const int t0 = blockIdx.x * RG_TOKENS, b = blockIdx.y;
    const int outs = blockDim.x / KS;
    const int slice = threadIdx.x / outs, ol = threadIdx.x % outs;
    const int o = blockIdx.z * outs + ol;
    const int n_t = min(RG_TOKENS, n_tokens - t0);
    for (int e = threadIdx.x; e < RG_TOKENS * bs; e += blockDim.x) {
        const int k = e / bs, i = e % bs;
        u_lds[i * RG_TOKENS + k] = k < n_t ? u[(size_t)(t0 + k) * width + (size_t)b * bs + i] : 0.f;
    }
    __syncthreads();
    if (KS == 1 && o >= bs) return;
    float acc_a[RG_TOKENS], acc_i[RG_TOKENS];
#pragma unroll
    for (int k = 0; k < RG_TOKENS; ++k) { acc_a[k] = 0.f; acc_i[k] = 0.f; }
    const int per = (bs + KS - 1) / KS;
    const int i0 = slice * per, i1 = min(bs, i0 + per);
    if (o < bs) {
        const float* wa = wa_t + (size_t)b * bs * bs + o;
        const float* wi = wi_t + (size_t)b * bs * bs + o;
#pragma unroll 4
        for (int i = i0; i < i1; ++i) {
            const float va = wa[(size_t)i * bs], vi = wi[(size_t)i * bs];
            const float4 u0 = *reinterpret_cast<const float4*>(u_lds + i * RG_TOKENS), u1 = *reinterpret_cast<const float4*>(u_lds + i * RG_TOKENS + 4);
            const float uv[RG_TOKENS] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
            for (int k = 0; k < RG_TOKENS; ++k) {
                acc_a[k] = fmaf(va, uv[k], acc_a[k]);
                acc_i[k] = fmaf(vi, uv[k], acc_i[k]);
            }
        }
    }
    if (KS > 1) {
        float* red = u_lds + (size_t)bs * RG_TOKENS;
#pragma unroll
        for (int k = 0; k < RG_TOKENS; ++k) {
            red[((slice * 2 + 0) * RG_TOKENS + k) * outs + ol] = acc_a[k];
            red[((slice * 2 + 1) * RG_TOKENS + k) * outs + ol] = acc_i[k];
        }
        __syncthreads();
        if (o >= bs || slice >= n_t) return;
        float sa = 0.f, si = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            sa += red[((s * 2 + 0) * RG_TOKENS + slice) * outs + ol];
            si += red[((s * 2 + 1) * RG_TOKENS + slice) * outs + ol];
        }
        acc_a[0] = sa; acc_i[0] = si;
    }
    const int ch = b * bs + o;
    const float c8 = decay_c[ch], bav = ba[ch], biv = bi[ch];
#pragma unroll
    for (int kk = 0; kk < (KS > 1 ? 1 : RG_TOKENS); ++kk) {
        const int k = KS > 1 ? slice : kk;
        if (k >= n_t) break;
        const float r = sigmoid_f(acc_a[kk] + bav), gate = sigmoid_f(acc_i[kk] + biv);
        const float log_a = c8 * r;
        const float a = expf(log_a);
        const float mult = sqrtf(fmaxf(-expm1f(2.f * log_a), 0.f));          // sqrt(1 - a^2), formed without the difference of near-equal numbers
        const size_t at = (size_t)(t0 + k) * width + ch;
        a_out[at] = a;
        g_out[at] = mult * gate * u_lds[o * RG_TOKENS + k];
    }
}

// ---- the linear recurrence S_t = a_t S_(t-1) + g_t, a thread per (sequence, channel) -------------------------------------
// out_t = S_t * gelu_tanh(y_t + y_bias): the other branch of the block rides along.
template <typename TA>
__global__ __launch_bounds__(256)
void linear_scan_kernel(const float* __restrict__ a, const float* __restrict__ g, const TA* __restrict__ y, long long y_stride,
                        const float* __restrict__ y_bias, float* __restrict__ state, long long state_stride, const int32_t* __restrict__ cu,
                        const int32_t* __restrict__ seq_new, const int32_t* __restrict__ seq_slot, TA* __restrict__ out, int width) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= width) return;
    const int n = seq_new[s], t0 = cu[s];
    if (n <= 0) return;
    float* st = state + (size_t)seq_slot[s] * state_stride + c;
    const float yb = y_bias ? y_bias[c] : 0.f;
    float S = *st;
    for (int j = 0; j < n; ++j) {
        const size_t at = (size_t)(t0 + j) * width + c;
        S = fmaf(a[at], S, g[at]);
        const float yv = gelu_tanh_f(to_float(y[(size_t)(t0 + j) * y_stride + c]) + yb);
        out[at] = from_float<TA>(S * yv);
    }
    *st = S;
}

// ---- the selective state-space recurrence --------------------------------------------------------------------------
// A wave per (sequence, head, 16 columns of the head's values).  Lane = 16 * slice + column: a lane keeps the state's rows
// n = slice, slice + 4, ... of its column in registers, NK of them.  xbc: the convolution's output [tokens][inner + 2 G N]
// as [x | B | C].  The state of a slot: [heads][N][P].
template <typename TA, int NK>
__global__ __launch_bounds__(64)
void ssm_scan_kernel(const float* __restrict__ xbc, long long xbc_stride, const TA* __restrict__ dt_raw, long long dt_stride,
                     const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
                     long long state_stride, const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_new, const int32_t* __restrict__ seq_slot,
                     float* __restrict__ y_out, int heads, int groups, int n_state, int p_dim) {
    const int s = blockIdx.z, h = blockIdx.y;
    const int lane = threadIdx.x, col = lane & 15, slice = lane >> 4;
    const int p = blockIdx.x * 16 + col;
    const int n = seq_new[s], t0 = cu[s];
    if (n <= 0) return;
    const int inner = heads * p_dim, grp = h / (heads / groups);
    const bool live = p < p_dim;
    float* st = state + (size_t)seq_slot[s] * state_stride + (size_t)h * n_state * p_dim;
    float S[NK];
#pragma unroll
    for (int k = 0; k < NK; ++k) {
        const int row = slice + 4 * k;
        S[k] = (live && row < n_state) ? st[(size_t)row * p_dim + p] : 0.f;
    }
    const float rate = -expf(a_log[h]), db = dt_bias[h], dsk = d_skip[h];
    for (int j = 0; j < n; ++j) {
        const size_t t = (size_t)(t0 + j);
        const float* row = xbc + t * xbc_stride;
        const float dt = softplus_f(to_float(dt_raw[t * dt_stride + h]) + db);
        const float decay = expf(rate * dt);
        const float xv = live ? row[(size_t)h * p_dim + p] : 0.f;
        const float dx = dt * xv;
        const float* Bv = row + inner + (size_t)grp * n_state;
        const float* Cv = row + inner + (size_t)groups * n_state + (size_t)grp * n_state;
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < NK; ++k) {
            const int r = slice + 4 * k;
            if (r < n_state) {
                S[k] = fmaf(decay, S[k], Bv[r] * dx);
                acc = fmaf(S[k], Cv[r], acc);
            }
        }
        acc += __shfl_xor(acc, 16, TQK_WAVE);
        acc += __shfl_xor(acc, 32, TQK_WAVE);
        if (live && slice == 0) y_out[t * inner + (size_t)h * p_dim + p] = fmaf(dsk, xv, acc);
    }
#pragma unroll
    for (int k = 0; k < NK; ++k) {
        const int row = slice + 4 * k;
        if (live && row < n_state) st[(size_t)row * p_dim + p] = S[k];
    }
}

// ---- long steps: the recurrences in chunks ---------------------------------------------------------------------------
// A step that brings many tokens of a sequence is cut into chunks of consecutive tokens of one sequence (chunk c: packed rows
// chunk_row0[c] .. + chunk_count[c]; the chunks of sequence s are seq_first[s] .. seq_first[s + 1], in order).  Three launches:
// every chunk runs its recurrence from a zero state and leaves its last state and the product of its decays; a carry pass walks a
// sequence's chunks in order, S <- decay S + local, and leaves in each chunk's place the state the chunk starts from (the
// sequence's state row gets the last one); every chunk runs again from that state and writes the outputs.  Twice the arithmetic,
// but as many independent pieces of work as there are chunks, where the plain kernels above have one per sequence.
enum { CHUNK_LOCAL = 1, CHUNK_APPLY = 2 };

template <typename TA, int MODE>
__global__ __launch_bounds__(256)
void linear_chunk_kernel(const float* __restrict__ a, const float* __restrict__ g, const TA* __restrict__ y, long long y_stride,
                         const float* __restrict__ y_bias, const int32_t* __restrict__ chunk_row0, const int32_t* __restrict__ chunk_count,
                         float* __restrict__ chunk_p, float* __restrict__ chunk_l, TA* __restrict__ out, int width) {
    const int c = blockIdx.y;
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= width) return;
    const int t0 = chunk_row0[c], n = chunk_count[c];
    float S = MODE == CHUNK_APPLY ? chunk_l[(size_t)c * width + ch] : 0.f, P = 1.f;
    const float yb = (MODE == CHUNK_APPLY && y_bias) ? y_bias[ch] : 0.f;
    for (int j = 0; j < n; ++j) {
        const size_t at = (size_t)(t0 + j) * width + ch;
        const float av = a[at];
        S = fmaf(av, S, g[at]);
        if (MODE == CHUNK_LOCAL) P *= av;
        else out[at] = from_float<TA>(S * gelu_tanh_f(to_float(y[(size_t)(t0 + j) * y_stride + ch]) + yb));
    }
    if (MODE == CHUNK_LOCAL) {
        chunk_p[(size_t)c * width + ch] = P;
        chunk_l[(size_t)c * width + ch] = S;
    }
}

// elements: per sequence `per_seq` state values; element e of a chunk decays with chunk_p[c * p_stride + e / p_div]
__global__ __launch_bounds__(256)
void chunk_carry_kernel(const float* __restrict__ chunk_p, long long p_stride, int p_div, float* __restrict__ chunk_l, const int32_t* __restrict__ seq_first,
                        const int32_t* __restrict__ seq_slot, float* __restrict__ state, long long state_stride, long long per_seq) {
    const int s = blockIdx.y;
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= per_seq) return;
    const int c0 = seq_first[s], c1 = seq_first[s + 1];
    if (c1 <= c0) return;
    float* st = state + (size_t)seq_slot[s] * state_stride + e;
    float S = *st;
    for (int c = c0; c < c1; ++c) {
        float* l = chunk_l + (size_t)c * per_seq + e;
        const float local = *l;
        *l = S;
        S = fmaf(chunk_p[(size_t)c * p_stride + e / p_div], S, local);
    }
    *st = S;
}

// dt = softplus(raw + bias) and the decay exp(-exp(a_log) dt) of every (token, head), once
template <typename TA>
__global__ __launch_bounds__(256)
void ssm_steps_kernel(const TA* __restrict__ dt_raw, long long dt_stride, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                      float* __restrict__ dt_out, float* __restrict__ decay_out, long long n, int heads) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long t = i / heads;
    const int h = (int)(i % heads);
    const float dt = softplus_f(to_float(dt_raw[t * dt_stride + h]) + dt_bias[h]);
    dt_out[i] = dt;
    decay_out[i] = expf(-expf(a_log[h]) * dt);
}

__device__ __forceinline__ float dpp_quad_xor1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false)); }
__device__ __forceinline__ float dpp_quad_xor2(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false)); }
__device__ __forceinline__ float dpp_half_mirror(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false)); }
__device__ __forceinline__ float dpp_row_mirror(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false)); }
// the sum over a row of 16 lanes, in every lane of the row, in one fixed order
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_quad_xor1(v);
    v += dpp_quad_xor2(v);
    v += dpp_half_mirror(v);
    v += dpp_row_mirror(v);
    return v;
}

// A block of four waves per (chunk, head, 64 columns of the head's values); a wave takes 16 columns.  Lane = 16 * column group +
// row group: a lane keeps RN consecutive rows of 4 consecutive columns of the state, so a token costs it RN values each of B and
// C and 4 of x for 4 RN products; a column's output is summed over the 16 row groups, which are one row of lanes.
// vec: rows and columns fall into pieces of four floats at aligned places (the host says so).
template <int RN, int MODE>
__global__ __launch_bounds__(256)
void ssm_chunk_kernel(const float* __restrict__ xbc, long long xbc_stride, const float* __restrict__ dt, const float* __restrict__ decay,
                      const float* __restrict__ d_skip, const int32_t* __restrict__ chunk_row0, const int32_t* __restrict__ chunk_count,
                      float* __restrict__ chunk_state, float* __restrict__ chunk_decay, float* __restrict__ y_out, int heads, int groups,
                      int n_state, int p_dim, int vec) {
    const int c = blockIdx.z, h = blockIdx.y;
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int rowgroup = lane & 15, colgroup = lane >> 4;
    const int p0 = (blockIdx.x * 4 + wave) * 16 + colgroup * 4, r0 = rowgroup * RN;
    if ((blockIdx.x * 4 + wave) * 16 >= p_dim) return;
    const int t0 = chunk_row0[c], n = chunk_count[c];
    const int inner = heads * p_dim, grp = h / (heads / groups);
    float* cs = chunk_state + ((size_t)c * heads + h) * n_state * p_dim;
    float S[RN][4];
#pragma unroll
    for (int i = 0; i < RN; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            S[i][j] = (MODE == CHUNK_APPLY && r0 + i < n_state && p0 + j < p_dim) ? cs[(size_t)(r0 + i) * p_dim + p0 + j] : 0.f;
    const float dsk = d_skip[h];
    float total = 1.f;
    for (int k = 0; k < n; ++k) {
        const size_t t = (size_t)(t0 + k);
        const float* row = xbc + t * xbc_stride;
        const float dtv = dt[t * heads + h], dec = decay[t * heads + h];
        const float* xs = row + (size_t)h * p_dim + p0;
        const float* Bs = row + inner + (size_t)grp * n_state + r0;
        const float* Cs = Bs + (size_t)groups * n_state;
        float x[4], B[RN], C[RN];
        if (vec) {
            const float4 xv = *reinterpret_cast<const float4*>(xs);
            x[0] = xv.x; x[1] = xv.y; x[2] = xv.z; x[3] = xv.w;
#pragma unroll
            for (int i = 0; i < RN; i += 4) {
                const float4 b = *reinterpret_cast<const float4*>(Bs + i);
                B[i] = b.x; B[i + 1 < RN ? i + 1 : i] = b.y; B[i + 2 < RN ? i + 2 : i] = b.z; B[i + 3 < RN ? i + 3 : i] = b.w;
                if (MODE == CHUNK_APPLY) {
                    const float4 cv = *reinterpret_cast<const float4*>(Cs + i);
                    C[i] = cv.x; C[i + 1 < RN ? i + 1 : i] = cv.y; C[i + 2 < RN ? i + 2 : i] = cv.z; C[i + 3 < RN ? i + 3 : i] = cv.w;
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) x[j] = p0 + j < p_dim ? xs[j] : 0.f;
#pragma unroll
            for (int i = 0; i < RN; ++i) {
                B[i] = r0 + i < n_state ? Bs[i] : 0.f;
                if (MODE == CHUNK_APPLY) C[i] = r0 + i < n_state ? Cs[i] : 0.f;
            }
        }
        float dx[4], acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) dx[j] = dtv * x[j];
#pragma unroll
        for (int i = 0; i < RN; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                S[i][j] = fmaf(dec, S[i][j], B[i] * dx[j]);
                if (MODE == CHUNK_APPLY) acc[j] = fmaf(S[i][j], C[i], acc[j]);
            }
        if (MODE == CHUNK_APPLY) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(dsk, x[j], row16_sum(acc[j]));
            if (rowgroup == 0) {
                float* yo = y_out + t * inner + (size_t)h * p_dim + p0;
                if (vec) *reinterpret_cast<float4*>(yo) = make_float4(acc[0], acc[1], acc[2], acc[3]);
                else
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (p0 + j < p_dim) yo[j] = acc[j];
            }
        } else total *= dec;
    }
    if (MODE == CHUNK_LOCAL) {
#pragma unroll
        for (int i = 0; i < RN; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (r0 + i < n_state && p0 + j < p_dim) cs[(size_t)(r0 + i) * p_dim + p0 + j] = S[i][j];
        if (blockIdx.x == 0 && threadIdx.x == 0) chunk_decay[(size_t)c * heads + h] = total;
    }
}

// ---- gate, then norm in parts --------------------------------------------------------------------------------
// v = y silu(z); every one of `parts` equal parts of a row is divided by its own root mean square; times w.  A block per
// (token, part).
template <typename TA>
__global__ __launch_bounds__(256)
void gated_part_norm_kernel(const float* __restrict__ y, const TA* __restrict__ z, long long z_stride, const float* __restrict__ w, float eps,
                            TA* __restrict__ out, int size, int part) {
    __shared__ float scratch[4];
    const int t = blockIdx.x, g = blockIdx.y;
    const float* yr = y + (size_t)t * size + (size_t)g * part;
    const TA* zr = z + (size_t)t * z_stride + (size_t)g * part;
    float ss = 0.f;
    for (int i = threadIdx.x; i < part; i += blockDim.x) {
        const float v = yr[i] * silu_f(to_float(zr[i]));
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
    for (int i = threadIdx.x; i < part; i += blockDim.x) {
        const float v = yr[i] * silu_f(to_float(zr[i]));
        out[(size_t)t * size + (size_t)g * part + i] = from_float<TA>(v * inv * w[(size_t)g * part + i]);
    }
}

__device__ __forceinline__ void store4(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void store4(bf16_t* p, const float (&v)[4]) {
    uint2 h;
    h.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
    h.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = h;
}

// The same where a part falls into aligned pieces of four values and a block's threads hold all of it: every value is read and
// gated once and waits in registers for the part's sum.
template <typename TA, int ITERS>
__global__ __launch_bounds__(1024)
void gated_part_norm_vec_kernel(const float* __restrict__ y, const TA* __restrict__ z, long long z_stride, const float* __restrict__ w, float eps,
                                TA* __restrict__ out, int size, int part) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, g = blockIdx.y;
    const float* yr = y + (size_t)t * size + (size_t)g * part;
    const TA* zr = z + (size_t)t * z_stride + (size_t)g * part;
    float v[ITERS][4];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int i = (it * blockDim.x + threadIdx.x) * 4;
        if (i < part) {
            float a[4], b[4];
            load4(yr + i, a);
            load4(zr + i, b);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[it][j] = a[j] * silu_f(b[j]);
                ss = fmaf(v[it][j], v[it][j], ss);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) v[it][j] = 0.f;
        }
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int i = (it * blockDim.x + threadIdx.x) * 4;
        if (i < part) {
            float wv[4], o[4];
            load4(w + (size_t)g * part + i, wv);
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = v[it][j] * inv * wv[j];
            store4(out + (size_t)t * size + (size_t)g * part + i, o);
        }
    }
}

// h += x, float32, element by element
__global__ __launch_bounds__(256)
void add_rows_kernel(float* __restrict__ h, const float* __restrict__ x, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) h[i] += x[i];
}

// ---- entry points ------------------------------------------------------------------------------------------------
extern "C" int tqk_conv_max_taps(void) { return TQK_CONV_MAX_TAPS; }
extern "C" int tqk_ssm_max_state(void) { return 256; }

extern "C" int tqk_conv_state(const void* x, int x_dtype, long long x_stride, const float* in_bias, const float* w, const float* bias, int taps,
                              int activation, const float* state, long long state_stride, const int32_t* tok_seq, const int32_t* tok_pos,
                              const int32_t* seq_slot, const int32_t* seq_start, float* out, int n_tokens, int channels, void* stream) {
    TQK_REQUIRE(x && w && state && tok_seq && tok_pos && seq_slot && seq_start && out, "tqk_conv_state: null pointer");
    TQK_REQUIRE(taps >= 1 && taps <= TQK_CONV_MAX_TAPS, "tqk_conv_state: %d taps, the kernel takes 1 to %d", taps, TQK_CONV_MAX_TAPS);
    TQK_REQUIRE(n_tokens >= 0 && channels > 0 && x_stride >= channels && state_stride >= (long long)(taps - 1) * channels,
                "tqk_conv_state: bad sizes");
    TQK_REQUIRE(activation == 0 || activation == 1, "tqk_conv_state: unknown activation %d", activation);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // steps of many rows whose rows fall into aligned pieces of four values: the kernel that keeps a window of rows in registers
    const size_t piece = 4 * (x_dtype == TQK_F32 ? 4 : 2);
    if (n_tokens >= 2 * CONV_ROWS && (x_dtype == TQK_F32 || x_dtype == TQK_BF16) && channels % 4 == 0 && x_stride % 4 == 0 &&
        (uintptr_t)x % piece == 0 && (uintptr_t)out % 16 == 0 && (n_tokens + CONV_ROWS - 1) / CONV_ROWS <= 65535) {
        dim3 grid((channels / 4 + 127) / 128, (n_tokens + CONV_ROWS - 1) / CONV_ROWS);
#define TQK_CONV(TA, TAPS) conv_state_vec_kernel<TA, TAPS><<<grid, 128, 0, s>>>((const TA*)x, x_stride, in_bias, w, bias, activation, state, state_stride, \
        tok_seq, tok_pos, seq_slot, seq_start, out, n_tokens, channels)
#define TQK_CONV_BY_TAPS(TA) switch (taps) { case 1: TQK_CONV(TA, 1); break; case 2: TQK_CONV(TA, 2); break; case 3: TQK_CONV(TA, 3); break; \
        case 4: TQK_CONV(TA, 4); break; case 5: TQK_CONV(TA, 5); break; case 6: TQK_CONV(TA, 6); break; case 7: TQK_CONV(TA, 7); break; \
        default: TQK_CONV(TA, 8); break; }
        if (x_dtype == TQK_F32) TQK_CONV_BY_TAPS(float) else TQK_CONV_BY_TAPS(bf16_t)
#undef TQK_CONV_BY_TAPS
#undef TQK_CONV
        return tqk_check_launch("tqk_conv_state");
    }
    // (the grid's second dimension takes 65535: longer steps go in pieces)
    for (int t0 = 0; t0 < n_tokens; t0 += 65535) {
        const int n = n_tokens - t0 < 65535 ? n_tokens - t0 : 65535;
        dim3 grid((channels + 255) / 256, n);
        if (x_dtype == TQK_F32)
            conv_state_kernel<float><<<grid, 256, 0, s>>>((const float*)x + (size_t)t0 * x_stride, x_stride, in_bias, w, bias, taps, activation, state, state_stride,
                                                          tok_seq + t0, tok_pos + t0, seq_slot, seq_start, out + (size_t)t0 * channels, channels);
        else if (x_dtype == TQK_BF16)
            conv_state_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x + (size_t)t0 * x_stride, x_stride, in_bias, w, bias, taps, activation, state, state_stride,
                                                           tok_seq + t0, tok_pos + t0, seq_slot, seq_start, out + (size_t)t0 * channels, channels);
        else return tqk_fail("tqk_conv_state: unknown dtype %d", x_dtype);
    }
    return tqk_check_launch("tqk_conv_state");
}

extern "C" int tqk_conv_state_update(const void* x, int x_dtype, long long x_stride, const float* in_bias, int taps, float* state, long long state_stride,
                                     const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, int n_seqs, int channels, void* stream) {
    TQK_REQUIRE(x && state && cu && seq_new && seq_slot, "tqk_conv_state_update: null pointer");
    TQK_REQUIRE(taps >= 1 && taps <= TQK_CONV_MAX_TAPS, "tqk_conv_state_update: %d taps, the kernel takes 1 to %d", taps, TQK_CONV_MAX_TAPS);
    TQK_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && channels > 0, "tqk_conv_state_update: bad sizes");
    if (n_seqs == 0 || taps == 1) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((channels + 255) / 256, n_seqs);
    if (x_dtype == TQK_F32)
        conv_state_update_kernel<float><<<grid, 256, 0, s>>>((const float*)x, x_stride, in_bias, taps, state, state_stride, cu, seq_new, seq_slot, channels);
    else if (x_dtype == TQK_BF16)
        conv_state_update_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, x_stride, in_bias, taps, state, state_stride, cu, seq_new, seq_slot, channels);
    else return tqk_fail("tqk_conv_state_update: unknown dtype %d", x_dtype);
    return tqk_check_launch("tqk_conv_state_update");
}

extern "C" int tqk_conv_state_step(const void* x, int x_dtype, long long x_stride, const float* in_bias, const float* w, const float* bias, int taps,
                                   int activation, float* state, long long state_stride, const int32_t* tok_seq, const int32_t* seq_slot, float* out,
                                   int n_tokens, int channels, void* stream) {
    TQK_REQUIRE(x && w && state && tok_seq && seq_slot && out, "tqk_conv_state_step: null pointer");
    TQK_REQUIRE(taps >= 1 && taps <= TQK_CONV_MAX_TAPS, "tqk_conv_state_step: %d taps, the kernel takes 1 to %d", taps, TQK_CONV_MAX_TAPS);
    TQK_REQUIRE(n_tokens >= 0 && n_tokens <= 65535 && channels > 0 && x_stride >= channels && state_stride >= (long long)(taps - 1) * channels,
                "tqk_conv_state_step: bad sizes");
    TQK_REQUIRE(activation == 0 || activation == 1, "tqk_conv_state_step: unknown activation %d", activation);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((channels + 255) / 256, n_tokens);
    if (x_dtype == TQK_F32)
        conv_state_step_kernel<float><<<grid, 256, 0, s>>>((const float*)x, x_stride, in_bias, w, bias, taps, activation, state, state_stride, tok_seq, seq_slot, out, channels);
    else if (x_dtype == TQK_BF16)
        conv_state_step_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, x_stride, in_bias, w, bias, taps, activation, state, state_stride, tok_seq, seq_slot, out, channels);
    else return tqk_fail("tqk_conv_state_step: unknown dtype %d", x_dtype);
    return tqk_check_launch("tqk_conv_state_step");
}

static int rglru_gates_launch(const float* u, const float* wa_t, const float* wi_t, const float* ba, const float* bi, const float* decay_c, float* a_out,
                              float* g_out, int n_tokens, int width, int blocks, int split, void* stream) {
    TQK_REQUIRE(u && wa_t && wi_t && ba && bi && decay_c && a_out && g_out, "tqk_rglru_gates: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && width > 0 && blocks > 0 && width % blocks == 0, "tqk_rglru_gates: width %d in %d blocks", width, blocks);
    const int bs = width / blocks;
    size_t lds = (size_t)RG_TOKENS * bs * sizeof(float);
    TQK_REQUIRE(lds <= 64 * 1024, "tqk_rglru_gates: blocks of %d channels, the kernel takes up to %d", bs, 64 * 1024 / (RG_TOKENS * 4));
    TQK_REQUIRE(blocks <= 65535, "tqk_rglru_gates: too many blocks for the grid");
    if (n_tokens == 0) return 0;
    const int groups = (n_tokens + RG_TOKENS - 1) / RG_TOKENS;
    // the inputs dealt out to slices where a thread per output would give the chip less than a wave per SIMD
    if (split && bs >= 2 * RG_TOKENS && bs <= 1024 && (long long)groups * blocks * ((bs + 63) / 64) < 1024) {
        const int outs = 256 / RG_TOKENS;
        lds += (size_t)RG_TOKENS * 2 * RG_TOKENS * outs * sizeof(float);
        dim3 grid(groups, blocks, (bs + outs - 1) / outs);
        rglru_gates_kernel<RG_TOKENS><<<grid, 256, lds, (hipStream_t)stream>>>(u, wa_t, wi_t, ba, bi, decay_c, a_out, g_out, n_tokens, width, bs);
        return tqk_check_launch("tqk_rglru_gates");
    }
    const int threads = bs >= 256 ? 256 : (bs + 63) / 64 * 64;
    dim3 grid(groups, blocks, (bs + threads - 1) / threads);
    rglru_gates_kernel<1><<<grid, threads, lds, (hipStream_t)stream>>>(u, wa_t, wi_t, ba, bi, decay_c, a_out, g_out, n_tokens, width, bs);
    return tqk_check_launch("tqk_rglru_gates");
}

extern "C" int tqk_rglru_gates(const float* u, const float* wa_t, const float* wi_t, const float* ba, const float* bi, const float* decay_c, float* a_out,
                               float* g_out, int n_tokens, int width, int blocks, void* stream) {
    return rglru_gates_launch(u, wa_t, wi_t, ba, bi, decay_c, a_out, g_out, n_tokens, width, blocks, 0, stream);
}

/* The same where the order of the sum over the inputs may depend on the step's size (steps of few tokens deal the inputs out to slices). */
extern "C" int tqk_rglru_gates_any_order(const float* u, const float* wa_t, const float* wi_t, const float* ba, const float* bi, const float* decay_c,
                                         float* a_out, float* g_out, int n_tokens, int width, int blocks, void* stream) {
    return rglru_gates_launch(u, wa_t, wi_t, ba, bi, decay_c, a_out, g_out, n_tokens, width, blocks, 1, stream);
}

extern "C" int tqk_linear_scan(const float* a, const float* g, const void* y, int act_dtype, long long y_stride, const float* y_bias, float* state,
                               long long state_stride, const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, void* out, int n_seqs,
                               int width, void* stream) {
    TQK_REQUIRE(a && g && y && state && cu && seq_new && seq_slot && out, "tqk_linear_scan: null pointer");
    TQK_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && width > 0 && y_stride >= width && state_stride >= width, "tqk_linear_scan: bad sizes");
    if (n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((width + 63) / 64, n_seqs);
    if (act_dtype == TQK_F32)
        linear_scan_kernel<float><<<grid, 64, 0, s>>>(a, g, (const float*)y, y_stride, y_bias, state, state_stride, cu, seq_new, seq_slot, (float*)out, width);
    else if (act_dtype == TQK_BF16)
        linear_scan_kernel<bf16_t><<<grid, 64, 0, s>>>(a, g, (const bf16_t*)y, y_stride, y_bias, state, state_stride, cu, seq_new, seq_slot, (bf16_t*)out, width);
    else return tqk_fail("tqk_linear_scan: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_linear_scan");
}

extern "C" int tqk_ssm_scan(const float* xbc, long long xbc_stride, const void* dt_raw, int dt_dtype, long long dt_stride, const float* dt_bias,
                            const float* a_log, const float* d_skip, float* state, long long state_stride, const int32_t* cu, const int32_t* seq_new,
                            const int32_t* seq_slot, float* y_out, int n_seqs, int heads, int groups, int n_state, int p_dim, void* stream) {
    TQK_REQUIRE(xbc && dt_raw && dt_bias && a_log && d_skip && state && cu && seq_new && seq_slot && y_out, "tqk_ssm_scan: null pointer");
    TQK_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && heads > 0 && heads <= 65535 && groups > 0 && heads % groups == 0 && n_state > 0 && p_dim > 0,
                "tqk_ssm_scan: bad sizes (%d heads in %d groups)", heads, groups);
    TQK_REQUIRE(n_state <= 256, "tqk_ssm_scan: a state of %d rows, the kernel takes up to 256", n_state);
    TQK_REQUIRE(xbc_stride >= (long long)heads * p_dim + 2LL * groups * n_state && state_stride >= (long long)heads * n_state * p_dim, "tqk_ssm_scan: strides too short");
    if (n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((p_dim + 15) / 16, heads, n_seqs);
#define TQK_SSM(TA, NK) ssm_scan_kernel<TA, NK><<<grid, 64, 0, s>>>(xbc, xbc_stride, (const TA*)dt_raw, dt_stride, dt_bias, a_log, d_skip, state, state_stride, \
        cu, seq_new, seq_slot, y_out, heads, groups, n_state, p_dim)
#define TQK_SSM_BY_SIZE(TA) do { if (n_state <= 64) TQK_SSM(TA, 16); else if (n_state <= 128) TQK_SSM(TA, 32); else TQK_SSM(TA, 64); } while (0)
    if (dt_dtype == TQK_F32) TQK_SSM_BY_SIZE(float);
    else if (dt_dtype == TQK_BF16) TQK_SSM_BY_SIZE(bf16_t);
    else return tqk_fail("tqk_ssm_scan: unknown dtype %d", dt_dtype);
#undef TQK_SSM_BY_SIZE
#undef TQK_SSM
    return tqk_check_launch("tqk_ssm_scan");
}

extern "C" int tqk_linear_chunks(const float* a, const float* g, const void* y, int act_dtype, long long y_stride, const float* y_bias,
                                 const int32_t* chunk_row0, const int32_t* chunk_count, int n_chunks, float* chunk_p, float* chunk_l, void* out, int mode,
                                 int width, void* stream) {
    TQK_REQUIRE(a && g && chunk_row0 && chunk_count && chunk_p && chunk_l, "tqk_linear_chunks: null pointer");
    TQK_REQUIRE(mode == CHUNK_LOCAL || (mode == CHUNK_APPLY && y && out && y_stride >= width), "tqk_linear_chunks: mode %d, or nothing to write to", mode);
    TQK_REQUIRE(n_chunks >= 0 && n_chunks <= 65535 && width > 0, "tqk_linear_chunks: bad sizes");
    if (n_chunks == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((width + 255) / 256, n_chunks);
#define TQK_LC(TA, MODE) linear_chunk_kernel<TA, MODE><<<grid, 256, 0, s>>>(a, g, (const TA*)y, y_stride, y_bias, chunk_row0, chunk_count, chunk_p, chunk_l, (TA*)out, width)
    if (mode == CHUNK_LOCAL) TQK_LC(float, CHUNK_LOCAL);
    else if (act_dtype == TQK_F32) TQK_LC(float, CHUNK_APPLY);
    else if (act_dtype == TQK_BF16) TQK_LC(bf16_t, CHUNK_APPLY);
    else return tqk_fail("tqk_linear_chunks: unknown dtype %d", act_dtype);
#undef TQK_LC
    return tqk_check_launch("tqk_linear_chunks");
}

extern "C" int tqk_chunk_carry(const float* chunk_p, long long p_stride, int p_div, float* chunk_l, const int32_t* seq_first, const int32_t* seq_slot,
                               float* state, long long state_stride, int n_seqs, long long per_seq, void* stream) {
    TQK_REQUIRE(chunk_p && chunk_l && seq_first && seq_slot && state, "tqk_chunk_carry: null pointer");
    TQK_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && per_seq > 0 && p_div > 0 && state_stride >= per_seq, "tqk_chunk_carry: bad sizes");
    if (n_seqs == 0) return 0;
    const long long blocks = (per_seq + 255) / 256;
    TQK_REQUIRE(blocks <= 0x7fffffff, "tqk_chunk_carry: too many elements");
    dim3 grid((unsigned)blocks, n_seqs);
    chunk_carry_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(chunk_p, p_stride, p_div, chunk_l, seq_first, seq_slot, state, state_stride, per_seq);
    return tqk_check_launch("tqk_chunk_carry");
}

extern "C" int tqk_ssm_steps(const void* dt_raw, int dt_dtype, long long dt_stride, const float* dt_bias, const float* a_log, float* dt_out,
                             float* decay_out, int n_tokens, int heads, void* stream) {
    TQK_REQUIRE(dt_raw && dt_bias && a_log && dt_out && decay_out, "tqk_ssm_steps: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && heads > 0 && dt_stride >= heads, "tqk_ssm_steps: bad sizes");
    const long long n = (long long)n_tokens * heads;
    if (n == 0) return 0;
    const long long blocks = (n + 255) / 256;
    TQK_REQUIRE(blocks <= 0x7fffffff, "tqk_ssm_steps: too many elements");
    hipStream_t s = (hipStream_t)stream;
    if (dt_dtype == TQK_F32) ssm_steps_kernel<float><<<(unsigned)blocks, 256, 0, s>>>((const float*)dt_raw, dt_stride, dt_bias, a_log, dt_out, decay_out, n, heads);
    else if (dt_dtype == TQK_BF16) ssm_steps_kernel<bf16_t><<<(unsigned)blocks, 256, 0, s>>>((const bf16_t*)dt_raw, dt_stride, dt_bias, a_log, dt_out, decay_out, n, heads);
    else return tqk_fail("tqk_ssm_steps: unknown dtype %d", dt_dtype);
    return tqk_check_launch("tqk_ssm_steps");
}

extern "C" int tqk_ssm_chunks(const float* xbc, long long xbc_stride, const float* dt, const float* decay, const float* d_skip, const int32_t* chunk_row0,
                              const int32_t* chunk_count, int n_chunks, float* chunk_state, float* chunk_decay, float* y_out, int mode, int heads,
                              int groups, int n_state, int p_dim, void* stream) {
    TQK_REQUIRE(xbc && dt && decay && d_skip && chunk_row0 && chunk_count && chunk_state && chunk_decay, "tqk_ssm_chunks: null pointer");
    TQK_REQUIRE(mode == CHUNK_LOCAL || (mode == CHUNK_APPLY && y_out), "tqk_ssm_chunks: mode %d, or nothing to write to", mode);
    TQK_REQUIRE(n_chunks >= 0 && n_chunks <= 65535 && heads > 0 && heads <= 65535 && groups > 0 && heads % groups == 0 && n_state > 0 && p_dim > 0,
                "tqk_ssm_chunks: bad sizes (%d heads in %d groups)", heads, groups);
    TQK_REQUIRE(n_state <= 256, "tqk_ssm_chunks: a state of %d rows, the kernel takes up to 256", n_state);
    TQK_REQUIRE(xbc_stride >= (long long)heads * p_dim + 2LL * groups * n_state, "tqk_ssm_chunks: stride too short");
    if (n_chunks == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int rn = n_state <= 16 ? 1 : n_state <= 32 ? 2 : n_state <= 64 ? 4 : n_state <= 128 ? 8 : 16;
    // pieces of four floats at aligned places: whole rows of four per lane, columns and the row's parts at multiples of four
    const int vec = (rn % 4 == 0 && n_state == 16 * rn && p_dim % 16 == 0 && xbc_stride % 4 == 0 && ((uintptr_t)xbc & 15) == 0 && ((uintptr_t)y_out & 15) == 0) ? 1 : 0;
    dim3 grid((p_dim + 63) / 64, heads, n_chunks);
#define TQK_SC(RN, MODE) ssm_chunk_kernel<RN, MODE><<<grid, 256, 0, s>>>(xbc, xbc_stride, dt, decay, d_skip, chunk_row0, chunk_count, chunk_state, chunk_decay, \
        y_out, heads, groups, n_state, p_dim, vec)
#define TQK_SC_BY_SIZE(MODE) do { if (rn == 1) TQK_SC(1, MODE); else if (rn == 2) TQK_SC(2, MODE); else if (rn == 4) TQK_SC(4, MODE); \
        else if (rn == 8) TQK_SC(8, MODE); else TQK_SC(16, MODE); } while (0)
    if (mode == CHUNK_LOCAL) TQK_SC_BY_SIZE(CHUNK_LOCAL); else TQK_SC_BY_SIZE(CHUNK_APPLY);
#undef TQK_SC_BY_SIZE
#undef TQK_SC
    return tqk_check_launch("tqk_ssm_chunks");
}

extern "C" int tqk_gated_part_norm(const float* y, const void* z, int act_dtype, long long z_stride, const float* w, float eps, void* out, int n_tokens,
                                   int size, int parts, void* stream) {
    TQK_REQUIRE(y && z && w && out, "tqk_gated_part_norm: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && size > 0 && parts > 0 && parts <= 65535 && size % parts == 0 && z_stride >= size, "tqk_gated_part_norm: %d values in %d parts", size, parts);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(n_tokens, parts);
    {
        const int part = size / parts, quads = part / 4;
        const size_t piece = act_dtype == TQK_F32 ? 16 : 8;
        const int threads = quads >= 1024 ? 1024 : (quads + 63) / 64 * 64;
        const int iters = threads > 0 ? (quads + threads - 1) / threads : 0;
        if ((act_dtype == TQK_F32 || act_dtype == TQK_BF16) && part % 4 == 0 && z_stride % 4 == 0 && iters >= 1 && iters <= 4 &&
            (((uintptr_t)y | (uintptr_t)w) & 15) == 0 && (((uintptr_t)z | (uintptr_t)out) % piece) == 0) {
#define TQK_GPN(TA, IT) gated_part_norm_vec_kernel<TA, IT><<<grid, threads, 0, s>>>(y, (const TA*)z, z_stride, w, eps, (TA*)out, size, part)
#define TQK_GPN_BY_ITERS(TA) do { if (iters == 1) TQK_GPN(TA, 1); else if (iters == 2) TQK_GPN(TA, 2); else TQK_GPN(TA, 4); } while (0)
            if (act_dtype == TQK_F32) TQK_GPN_BY_ITERS(float); else TQK_GPN_BY_ITERS(bf16_t);
#undef TQK_GPN_BY_ITERS
#undef TQK_GPN
            return tqk_check_launch("tqk_gated_part_norm");
        }
    }
    if (act_dtype == TQK_F32) gated_part_norm_kernel<float><<<grid, 256, 0, s>>>(y, (const float*)z, z_stride, w, eps, (float*)out, size, size / parts);
    else if (act_dtype == TQK_BF16) gated_part_norm_kernel<bf16_t><<<grid, 256, 0, s>>>(y, (const bf16_t*)z, z_stride, w, eps, (bf16_t*)out, size, size / parts);
    else return tqk_fail("tqk_gated_part_norm: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_gated_part_norm");
}

extern "C" int tqk_add_rows(float* h, const float* x, long long n, void* stream) {
    TQK_REQUIRE(h && x && n >= 0, "tqk_add_rows: null pointer");
    if (n == 0) return 0;
    const long long blocks = (n + 255) / 256;
    TQK_REQUIRE(blocks <= 0x7fffffff, "tqk_add_rows: too many elements");
    add_rows_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(h, x, n);
    return tqk_check_launch("tqk_add_rows");
}
