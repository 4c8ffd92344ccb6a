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

// ---- gates of the RG-LRU ---------------------------------------------------------------------------------
// The two gates' matrices are block-diagonal: `blocks` square matrices of bs = width / blocks.  wa_t and wi_t hold them
// with the input index first, [blocks][bs in][bs out], so that neighbouring threads read neighbouring outputs.  A block
// of threads takes RG_TOKENS tokens, one diagonal block and up to 256 of its outputs; the tokens' inputs wait in LDS.
// The sum over the inputs runs in their order, whatever else the step holds.
#define RG_TOKENS 8
__global__ __launch_bounds__(256)
void rglru_gates_kernel(const float* __restrict__ u, const float* __restrict__ wa_t, const float* __restrict__ wi_t, const float* __restrict__ ba,
                        const float* __restrict__ bi, const float* __restrict__ decay_c, float* __restrict__ a_out, float* __restrict__ g_out,
                        int n_tokens, int width, int bs) {
    extern __shared__ float u_lds[];                  // [RG_TOKENS][bs]
    const int t0 = blockIdx.x * RG_TOKENS, b = blockIdx.y;
    const int o = blockIdx.z * blockDim.x + threadIdx.x;
    const int n_t = min(RG_TOKENS, n_tokens - t0);
    for (int e = threadIdx.x; e < RG_TOKENS * bs; e += blockDim.x) {
        const int k = e / bs, i = e % bs;
        u_lds[e] = k < n_t ? u[(size_t)(t0 + k) * width + (size_t)b * bs + i] : 0.f;
    }
    __syncthreads();
    if (o >= bs) return;
    float acc_a[RG_TOKENS], acc_i[RG_TOKENS];
#pragma unroll
    for (int k = 0; k < RG_TOKENS; ++k) { acc_a[k] = 0.f; acc_i[k] = 0.f; }
    const float* wa = wa_t + (size_t)b * bs * bs + o;
    const float* wi = wi_t + (size_t)b * bs * bs + o;
    for (int i = 0; i < bs; ++i) {
        const float va = wa[(size_t)i * bs], vi = wi[(size_t)i * bs];
#pragma unroll
        for (int k = 0; k < RG_TOKENS; ++k) {
            const float uv = u_lds[k * bs + i];
            acc_a[k] = fmaf(va, uv, acc_a[k]);
            acc_i[k] = fmaf(vi, uv, acc_i[k]);
        }
    }
    const int ch = b * bs + o;
    const float c8 = decay_c[ch], bav = ba[ch], biv = bi[ch];
#pragma unroll
    for (int k = 0; k < RG_TOKENS; ++k) {
        if (k >= n_t) break;
        const float r = sigmoid_f(acc_a[k] + bav), gate = sigmoid_f(acc_i[k] + biv);
        const float log_a = c8 * r;
        const float a = expf(log_a);
        const float mult = sqrtf(fmaxf(-expm1f(2.f * log_a), 0.f));          // sqrt(1 - a^2), formed without the difference of near-equal numbers
        const size_t at = (size_t)(t0 + k) * width + ch;
        a_out[at] = a;
        g_out[at] = mult * gate * u_lds[k * bs + o];
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

extern "C" int tqk_rglru_gates(const float* u, const float* wa_t, const float* wi_t, const float* ba, const float* bi, const float* decay_c, float* a_out,
                               float* g_out, int n_tokens, int width, int blocks, void* stream) {
    TQK_REQUIRE(u && wa_t && wi_t && ba && bi && decay_c && a_out && g_out, "tqk_rglru_gates: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && width > 0 && blocks > 0 && width % blocks == 0, "tqk_rglru_gates: width %d in %d blocks", width, blocks);
    const int bs = width / blocks;
    const size_t lds = (size_t)RG_TOKENS * bs * sizeof(float);
    TQK_REQUIRE(lds <= 64 * 1024, "tqk_rglru_gates: blocks of %d channels, the kernel takes up to %d", bs, 64 * 1024 / (RG_TOKENS * 4));
    TQK_REQUIRE(blocks <= 65535, "tqk_rglru_gates: too many blocks for the grid");
    if (n_tokens == 0) return 0;
    const int threads = bs >= 256 ? 256 : (bs + 63) / 64 * 64;
    dim3 grid((n_tokens + RG_TOKENS - 1) / RG_TOKENS, blocks, (bs + threads - 1) / threads);
    rglru_gates_kernel<<<grid, threads, lds, (hipStream_t)stream>>>(u, wa_t, wi_t, ba, bi, decay_c, a_out, g_out, n_tokens, width, bs);
    return tqk_check_launch("tqk_rglru_gates");
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

extern "C" int tqk_gated_part_norm(const float* y, const void* z, int act_dtype, long long z_stride, const float* w, float eps, void* out, int n_tokens,
                                   int size, int parts, void* stream) {
    TQK_REQUIRE(y && z && w && out, "tqk_gated_part_norm: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && size > 0 && parts > 0 && parts <= 65535 && size % parts == 0 && z_stride >= size, "tqk_gated_part_norm: %d values in %d parts", size, parts);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(n_tokens, parts);
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
