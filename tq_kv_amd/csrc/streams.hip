// The residual stream in several copies, a layer norm with weight and bias, and the previous token mixed into what a mixer reads.
// float32 arithmetic throughout.
//
//   tqk_streams_fill    X[t, s] = h[t] for every copy s
//   tqk_streams_step    for every token, in one pass over its copies: first (where y is given) the update of all copies from the old ones,
//                       X'[t, r] = sum_s mix[s, r] X[t, s] + out[r] y[t]; then (where `in` is given) what the next part reads,
//                       u = sum_s in[s] X'[t, s], left as it is in u_out and / or normed, (u - mean) / sqrt(var + eps) w + b, in n_out.
//                       The variance is the mean of the squared deviations from the mean (two passes over a row kept in LDS).
//   tqk_add_layer_norm  out[i] = LN(h[rows[i]] + delta[rows[i]]) (rows null: row i; h or delta may be missing; write_back: h keeps the sum)
//   tqk_token_shift     out[t] = n[t] + (n[t - 1] - n[t]) mu, the row before a sequence's first token of the step taken from the
//                       sequence's state (zeros before its first token); `remember` (steps of one token a sequence) also leaves n[t] there
//   tqk_shift_remember  state of sequence s = n[last token the step brings of s]
//   tqk_normed_pair_sum out[t] = c (x[t] / rms(x[t]) wx + y[t] / rms(y[t]) wy)
#include "common.h"
#include "tq_kernels.h"

#define STREAMS_MAX 16

__global__ __launch_bounds__(256)
void streams_fill_kernel(const float* __restrict__ h, float* __restrict__ X, int S, int W) {
    const size_t t = blockIdx.x;
    for (int e = threadIdx.x; e < W; e += blockDim.x) {
        const float v = h[t * W + e];
        for (int s = 0; s < S; ++s) X[(t * S + s) * W + e] = v;
    }
}

// SMAX: the most copies this instance takes (the loops over the copies are unrolled up to it)
template <typename TY, typename TN, int SMAX>
__global__ __launch_bounds__(1024)
void streams_step_kernel(float* __restrict__ X, int S, const TY* __restrict__ y, const float* __restrict__ mix, const float* __restrict__ outw,
                         const float* __restrict__ in, const float* __restrict__ nw, const float* __restrict__ nb, float eps,
                         float* __restrict__ u_out, TN* __restrict__ n_out, int W) {
    extern __shared__ float row_u[];
    __shared__ float scratch[16];
    __shared__ float s_mix[STREAMS_MAX * STREAMS_MAX], s_out[STREAMS_MAX], s_in[STREAMS_MAX];
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x; i < S * S && y; i += blockDim.x) s_mix[i] = mix[i];
    if (threadIdx.x < S) {
        if (y) s_out[threadIdx.x] = outw[threadIdx.x];
        if (in) s_in[threadIdx.x] = in[threadIdx.x];
    }
    __syncthreads();
    float* xr = X + t * S * W;
    float sum = 0.f;
    for (int e = threadIdx.x; e < W; e += blockDim.x) {
        float x[SMAX];
#pragma unroll
        for (int s = 0; s < SMAX; ++s) x[s] = s < S ? xr[(size_t)s * W + e] : 0.f;
        if (y) {
            const float yv = to_float(y[t * W + e]);
            float nx[SMAX];
#pragma unroll
            for (int r = 0; r < SMAX; ++r) {
                float acc = 0.f;
                if (r < S) {
#pragma unroll
                    for (int s = 0; s < SMAX; ++s)
                        if (s < S) acc = fmaf(s_mix[s * S + r], x[s], acc);
                    acc = fmaf(s_out[r], yv, acc);
                    xr[(size_t)r * W + e] = acc;
                }
                nx[r] = acc;
            }
#pragma unroll
            for (int s = 0; s < SMAX; ++s) x[s] = nx[s];
        }
        if (in) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
                if (s < S) u = fmaf(s_in[s], x[s], u);
            row_u[e] = u;
            sum += u;
            if (u_out) u_out[t * W + e] = u;
        }
    }
    if (!in || !n_out) return;
    const float mean = block_sum(sum, scratch) / (float)W;
    float ss = 0.f;
    for (int e = threadIdx.x; e < W; e += blockDim.x) { const float dlt = row_u[e] - mean; ss = fmaf(dlt, dlt, ss); }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
    for (int e = threadIdx.x; e < W; e += blockDim.x) n_out[t * W + e] = from_float<TN>((row_u[e] - mean) * inv * nw[e] + nb[e]);
}

template <typename TD, typename TO>
__global__ __launch_bounds__(256)
void add_layer_norm_kernel(float* __restrict__ h, const TD* __restrict__ delta, const int32_t* __restrict__ rows, const float* __restrict__ w,
                           const float* __restrict__ b, float eps, TO* __restrict__ out, int W, int write_back) {
    extern __shared__ float row_u[];
    __shared__ float scratch[4];
    const size_t i = blockIdx.x, r = rows ? (size_t)rows[i] : i;
    float sum = 0.f;
    for (int e = threadIdx.x; e < W; e += blockDim.x) {
        float v = h ? h[r * W + e] : 0.f;
        if (delta) v += to_float(delta[r * W + e]);
        if (write_back && h) h[r * W + e] = v;
        row_u[e] = v;
        sum += v;
    }
    const float mean = block_sum(sum, scratch) / (float)W;
    float ss = 0.f;
    for (int e = threadIdx.x; e < W; e += blockDim.x) { const float dlt = row_u[e] - mean; ss = fmaf(dlt, dlt, ss); }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
    for (int e = threadIdx.x; e < W; e += blockDim.x) out[i * W + e] = from_float<TO>((row_u[e] - mean) * inv * w[e] + b[e]);
}

template <typename TO>
__global__ __launch_bounds__(256)
void token_shift_kernel(const float* __restrict__ n, const float* __restrict__ mu, float* __restrict__ state, long long state_stride,
                        const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ seq_start,
                        const int32_t* __restrict__ seq_slot, TO* __restrict__ out, int W, int remember) {
    const size_t t = blockIdx.x;
    const int seq = tok_seq[t];
    const bool inside = tok_pos[t] > seq_start[seq];
    float* st = state + (size_t)seq_slot[seq] * state_stride;
    for (int e = threadIdx.x; e < W; e += blockDim.x) {
        const float cur = n[t * W + e];
        const float prev = inside ? n[(t - 1) * W + e] : st[e];
        out[t * W + e] = from_float<TO>(cur + (prev - cur) * mu[e]);
        if (remember) st[e] = cur;
    }
}

__global__ __launch_bounds__(256)
void shift_remember_kernel(const float* __restrict__ n, float* __restrict__ state, long long state_stride, const int32_t* __restrict__ cu,
                           const int32_t* __restrict__ seq_new, const int32_t* __restrict__ seq_slot, int W) {
    const int s = blockIdx.x;
    if (seq_new[s] <= 0) return;
    const size_t t = (size_t)cu[s] + seq_new[s] - 1;
    float* st = state + (size_t)seq_slot[s] * state_stride;
    for (int e = threadIdx.x; e < W; e += blockDim.x) st[e] = n[t * W + e];
}

extern "C" int tqk_streams_max(void) { return STREAMS_MAX; }

extern "C" int tqk_streams_fill(const float* h, float* X, int n_streams, int n_tokens, int width, void* stream) {
    TQK_REQUIRE(h && X, "tqk_streams_fill: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_streams > 0 && width > 0, "tqk_streams_fill: bad sizes");
    if (n_tokens == 0) return 0;
    streams_fill_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(h, X, n_streams, width);
    return tqk_check_launch("tqk_streams_fill");
}

extern "C" int tqk_streams_step(float* X, int n_streams, const void* y, int y_dtype, const float* mix, const float* out_w, const float* in_w,
                                const float* norm_w, const float* norm_b, float eps, float* u_out, void* n_out, int n_dtype, int n_tokens, int width,
                                int wide, void* stream) {
    TQK_REQUIRE(X, "tqk_streams_step: null pointer");
    TQK_REQUIRE(n_streams > 0 && n_streams <= STREAMS_MAX, "tqk_streams_step: %d copies of the stream, the kernel takes up to %d", n_streams, STREAMS_MAX);
    TQK_REQUIRE(!y || (mix && out_w), "tqk_streams_step: an update without its weights");
    TQK_REQUIRE(!n_out || (in_w && norm_w && norm_b), "tqk_streams_step: a norm without its weights");
    TQK_REQUIRE(!u_out || in_w, "tqk_streams_step: a sum without its weights");
    TQK_REQUIRE(n_tokens >= 0 && width > 0 && width <= 12288, "tqk_streams_step: bad sizes");
    if (n_tokens == 0 || (!y && !in_w)) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)width * sizeof(float);
    // wide (steps of few tokens, where the caller does not need one order of a row's sums for every kind of step): four times the
    // threads a row, so that a thread has a quarter of the loads to wait for one after the other
    const int threads = wide && width >= 1024 ? 1024 : 256;
#define TQK_SS_N(TY, TN, SMAX) streams_step_kernel<TY, TN, SMAX><<<n_tokens, threads, lds, s>>>(X, n_streams, (const TY*)y, mix, out_w, in_w, norm_w, norm_b, eps, u_out, (TN*)n_out, width)
#define TQK_SS(TY, TN) do { if (n_streams <= 1) TQK_SS_N(TY, TN, 1); else if (n_streams <= 2) TQK_SS_N(TY, TN, 2); else if (n_streams <= 4) TQK_SS_N(TY, TN, 4); \
        else if (n_streams <= 8) TQK_SS_N(TY, TN, 8); else TQK_SS_N(TY, TN, STREAMS_MAX); } while (0)
    const int yd = y ? y_dtype : TQK_F32, nd = n_out ? n_dtype : TQK_F32;
    if (yd == TQK_F32 && nd == TQK_F32) TQK_SS(float, float);
    else if (yd == TQK_F32 && nd == TQK_BF16) TQK_SS(float, bf16_t);
    else if (yd == TQK_BF16 && nd == TQK_F32) TQK_SS(bf16_t, float);
    else if (yd == TQK_BF16 && nd == TQK_BF16) TQK_SS(bf16_t, bf16_t);
    else return tqk_fail("tqk_streams_step: unknown dtypes %d, %d", y_dtype, n_dtype);
#undef TQK_SS
#undef TQK_SS_N
    return tqk_check_launch("tqk_streams_step");
}

extern "C" int tqk_add_layer_norm(float* h, const void* delta, int delta_dtype, const int32_t* rows, int n_rows, const float* weight, const float* bias,
                                  float eps, void* out, int out_dtype, int width, int write_back, void* stream) {
    TQK_REQUIRE((h || delta) && weight && bias && out, "tqk_add_layer_norm: null pointer");
    TQK_REQUIRE(n_rows >= 0 && width > 0 && width <= 12288, "tqk_add_layer_norm: bad sizes");
    TQK_REQUIRE(!(write_back && rows), "tqk_add_layer_norm: chosen rows are not written back");
    if (n_rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)width * sizeof(float);
#define TQK_ALN(TD, TO) add_layer_norm_kernel<TD, TO><<<n_rows, 256, lds, s>>>(h, (const TD*)delta, rows, weight, bias, eps, (TO*)out, width, write_back)
    const int dd = delta ? delta_dtype : TQK_F32;
    if (dd == TQK_F32 && out_dtype == TQK_F32) TQK_ALN(float, float);
    else if (dd == TQK_F32 && out_dtype == TQK_BF16) TQK_ALN(float, bf16_t);
    else if (dd == TQK_BF16 && out_dtype == TQK_F32) TQK_ALN(bf16_t, float);
    else if (dd == TQK_BF16 && out_dtype == TQK_BF16) TQK_ALN(bf16_t, bf16_t);
    else return tqk_fail("tqk_add_layer_norm: unknown dtypes %d, %d", delta_dtype, out_dtype);
#undef TQK_ALN
    return tqk_check_launch("tqk_add_layer_norm");
}

extern "C" int tqk_token_shift(const float* n, const float* mu, float* state, long long state_stride, const int32_t* tok_seq, const int32_t* tok_pos,
                               const int32_t* seq_start, const int32_t* seq_slot, void* out, int out_dtype, int n_tokens, int width, int remember,
                               void* stream) {
    TQK_REQUIRE(n && mu && state && tok_seq && tok_pos && seq_start && seq_slot && out, "tqk_token_shift: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && width > 0 && state_stride >= width, "tqk_token_shift: bad sizes");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == TQK_F32) token_shift_kernel<float><<<n_tokens, 256, 0, s>>>(n, mu, state, state_stride, tok_seq, tok_pos, seq_start, seq_slot, (float*)out, width, remember);
    else if (out_dtype == TQK_BF16) token_shift_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(n, mu, state, state_stride, tok_seq, tok_pos, seq_start, seq_slot, (bf16_t*)out, width, remember);
    else return tqk_fail("tqk_token_shift: unknown dtype %d", out_dtype);
    return tqk_check_launch("tqk_token_shift");
}

extern "C" int tqk_shift_remember(const float* n, float* state, long long state_stride, const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot,
                                  int n_seqs, int width, void* stream) {
    TQK_REQUIRE(n && state && cu && seq_new && seq_slot, "tqk_shift_remember: null pointer");
    TQK_REQUIRE(n_seqs >= 0 && width > 0 && state_stride >= width, "tqk_shift_remember: bad sizes");
    if (n_seqs == 0) return 0;
    shift_remember_kernel<<<n_seqs, 256, 0, (hipStream_t)stream>>>(n, state, state_stride, cu, seq_new, seq_slot, width);
    return tqk_check_launch("tqk_shift_remember");
}

// out[t] = c (x[t] / rms(x[t]) wx + y[t] / rms(y[t]) wy): the outputs of two parts that ran side by side, each normed over the row
template <typename TA, typename TO>
__global__ __launch_bounds__(256)
void normed_pair_sum_kernel(const TA* __restrict__ x, const TA* __restrict__ y, const float* __restrict__ wx, const float* __restrict__ wy, float eps,
                            float c, TO* __restrict__ out, int W) {
    __shared__ float scratch[4];
    const size_t t = blockIdx.x;
    float sx = 0.f, sy = 0.f;
    for (int e = threadIdx.x; e < W; e += blockDim.x) {
        const float a = to_float(x[t * W + e]), b = to_float(y[t * W + e]);
        sx = fmaf(a, a, sx);
        sy = fmaf(b, b, sy);
    }
    const float ix = 1.f / sqrtf(block_sum(sx, scratch) / (float)W + eps);
    const float iy = 1.f / sqrtf(block_sum(sy, scratch) / (float)W + eps);
    for (int e = threadIdx.x; e < W; e += blockDim.x)
        out[t * W + e] = from_float<TO>(c * (to_float(x[t * W + e]) * ix * wx[e] + to_float(y[t * W + e]) * iy * wy[e]));
}

extern "C" int tqk_normed_pair_sum(const void* x, const void* y, int dtype, const float* wx, const float* wy, float eps, float c, void* out, int out_dtype,
                                   int n_tokens, int width, void* stream) {
    TQK_REQUIRE(x && y && wx && wy && out, "tqk_normed_pair_sum: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && width > 0, "tqk_normed_pair_sum: bad sizes");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TQK_NPS(TA, TO) normed_pair_sum_kernel<TA, TO><<<n_tokens, 256, 0, s>>>((const TA*)x, (const TA*)y, wx, wy, eps, c, (TO*)out, width)
    if (dtype == TQK_F32 && out_dtype == TQK_F32) TQK_NPS(float, float);
    else if (dtype == TQK_BF16 && out_dtype == TQK_BF16) TQK_NPS(bf16_t, bf16_t);
    else if (dtype == TQK_BF16 && out_dtype == TQK_F32) TQK_NPS(bf16_t, float);
    else if (dtype == TQK_F32 && out_dtype == TQK_BF16) TQK_NPS(float, bf16_t);
    else return tqk_fail("tqk_normed_pair_sum: unknown dtypes %d, %d", dtype, out_dtype);
#undef TQK_NPS
    return tqk_check_launch("tqk_normed_pair_sum");
}
