// Attention whose heads have values of another size than their keys, with what some designs put
// around the softmax: a norm of every query and key head before the rotation, values mixed with
// those of an earlier layer, a cap on the scores, a window that keeps a sequence's first
// positions, and a sink in the softmax's denominator.  float32 arithmetic throughout, any sizes;
// the kernels for the matrix cores are in attention_masked_mfma.hip.
//
//   q_h <- rot(q_h / rms(q_h) * w_q),  k_g <- rot(k_g / rms(k_g) * w_k)      (rms with eps inside the root)
//   v_g <- (1 - lambda) v_g + lambda v'_g                                      (v' another layer's values of the token)
//   s_ij = scale q_i . k_j;  s_ij <- cap tanh(s_ij / cap)
//   i sees j  iff  j <= i and (window == 0 or i - j < window or j < keep_first)
//   p_ij = exp(s_ij) / (sum_j' exp(s_ij') + exp(sink_h))
//
// Cache pages: keys [kv head][position][key_dim], values [kv head][value_dim][place of the position]
// (value_place in common.h).
#include "common.h"
#include "tq_kernels.h"

#define AM_WAVES 4
#define AM_MAX_D 256

// ---- norm of heads, rotation, value mixing, cache write ---------------------------------------------
// A wave per head of a token: heads 0..H-1 are queries, then G key heads, then G value heads; a row of qkv is
// [H * dk | G * dk | G * dv].
template <typename TA, typename TW>
__global__ __launch_bounds__(AM_WAVES * TQK_WAVE)
void normed_rope_store_kernel(const TA* __restrict__ qkv, const TW* __restrict__ q_norm_w, const TW* __restrict__ k_norm_w, float eps,
                              const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot_dim, int max_positions,
                              const TW* __restrict__ mix, const TA* __restrict__ mix_with, TA* __restrict__ mix_keep,
                              const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                              const int32_t* __restrict__ page_table, int table_width, TA* __restrict__ keys, TA* __restrict__ values,
                              TA* __restrict__ q_out, int n_heads, int n_kv_heads, int dk, int dv, int write_kv) {
    const int t = blockIdx.x;
    const int head = blockIdx.y * AM_WAVES + threadIdx.x / TQK_WAVE;
    const int lane = threadIdx.x % TQK_WAVE;
    if (head >= n_heads + 2 * n_kv_heads) return;
    const int pos = tok_pos[t];
    const int kind = head < n_heads ? 0 : (head < n_heads + n_kv_heads ? 1 : 2);
    if (kind != 0 && !write_kv) return;
    const size_t total = (size_t)(n_heads + n_kv_heads) * dk + (size_t)n_kv_heads * dv;
    const TA* row = qkv + (size_t)t * total;
    int page = -1;
    if (kind != 0) {
        page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
        if (page < 0) return;                          // the host never lets this happen
    }
    if (kind == 2) {
        const int g = head - n_heads - n_kv_heads;
        const TA* src = row + (size_t)(n_heads + n_kv_heads) * dk + (size_t)g * dv;
        TA* dst = values + ((size_t)page * n_kv_heads + g) * TQK_PAGE * dv + value_place(pos % TQK_PAGE);
        const float lam = mix && mix_with ? to_float(mix[0]) : 0.f;
        for (int i = lane; i < dv; i += TQK_WAVE) {
            float v = to_float(src[i]);
            const size_t at = ((size_t)t * n_kv_heads + g) * dv + i;
            if (mix_with) v = (1.f - lam) * v + lam * to_float(mix_with[at]);
            const TA stored = from_float<TA>(v);
            if (mix_keep) mix_keep[at] = stored;
            dst[(size_t)i * TQK_PAGE] = stored;
        }
        return;
    }
    const TA* src = row + (size_t)head * dk;
    const TW* w = kind == 0 ? q_norm_w : k_norm_w;
    float inv = 1.f;
    if (w) {
        float ss = 0.f;
        for (int i = lane; i < dk; i += TQK_WAVE) { const float v = to_float(src[i]); ss = fmaf(v, v, ss); }
        inv = 1.f / sqrtf(wave_sum(ss) / (float)dk + eps);
    }
    TA* dst = kind == 0 ? q_out + ((size_t)t * n_heads + head) * dk
                        : keys + (((size_t)page * n_kv_heads + (head - n_heads)) * TQK_PAGE + pos % TQK_PAGE) * dk;
    const int half = rot_dim / 2;
    const bool rotate = rot_dim > 0 && pos < max_positions;
    for (int i = lane; i < dk; i += TQK_WAVE) {
        float x = to_float(src[i]) * inv * (w ? to_float(w[i]) : 1.f);
        if (rotate && i < rot_dim) {
            const bool first = i < half;
            const int p = first ? i : i - half, partner = first ? i + half : i - half;
            const float y = to_float(src[partner]) * inv * (w ? to_float(w[partner]) : 1.f);
            const float c = cos_table[(size_t)pos * half + p], s = sin_table[(size_t)pos * half + p];
            x = first ? x * c - y * s : x * c + y * s;
        }
        dst[i] = from_float<TA>(x);
    }
}

// ---- bias, rotation, then a norm without a weight, cache write ------------------------------------------
// What another family of designs does with its heads: the projections' biases are added, q and k are turned (in halves,
// style 1, or in neighbouring pairs, style 2: element 2i with 2i + 1), and only then every query and key head is divided
// by its root mean square (normed != 0; no weight).  A wave per head of a token, as above; a lane keeps its elements
// (up to AM_MAX_D / 64) between the sum of squares and the store.
template <typename TA, typename TB>
__global__ __launch_bounds__(AM_WAVES * TQK_WAVE)
void rope_norm_store_kernel(const TA* __restrict__ qkv, const TB* __restrict__ bias, const float* __restrict__ cos_table,
                            const float* __restrict__ sin_table, int rot_dim, int style, int max_positions, int normed, float eps,
                            const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table,
                            int table_width, TA* __restrict__ keys, TA* __restrict__ values, TA* __restrict__ q_out, int n_heads, int n_kv_heads,
                            int dk, int dv, int write_kv) {
    const int t = blockIdx.x;
    const int head = blockIdx.y * AM_WAVES + threadIdx.x / TQK_WAVE;
    const int lane = threadIdx.x % TQK_WAVE;
    if (head >= n_heads + 2 * n_kv_heads) return;
    const int pos = tok_pos[t];
    const int kind = head < n_heads ? 0 : (head < n_heads + n_kv_heads ? 1 : 2);
    if (kind != 0 && !write_kv) return;
    const size_t total = (size_t)(n_heads + n_kv_heads) * dk + (size_t)n_kv_heads * dv;
    const TA* row = qkv + (size_t)t * total;
    int page = -1;
    if (kind != 0) {
        page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
        if (page < 0) return;                          // the host never lets this happen
    }
    if (kind == 2) {
        const int g = head - n_heads - n_kv_heads;
        const size_t off = (size_t)(n_heads + n_kv_heads) * dk + (size_t)g * dv;
        TA* dst = values + ((size_t)page * n_kv_heads + g) * TQK_PAGE * dv + value_place(pos % TQK_PAGE);
        for (int i = lane; i < dv; i += TQK_WAVE)
            dst[(size_t)i * TQK_PAGE] = from_float<TA>(to_float(row[off + i]) + (bias ? to_float(bias[off + i]) : 0.f));
        return;
    }
    const size_t off = (size_t)head * dk;
    const int half = rot_dim / 2;
    const bool rotate = rot_dim > 0 && style != 0 && pos < max_positions;
    float x[AM_MAX_D / TQK_WAVE];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < AM_MAX_D / TQK_WAVE; ++k) {
        const int i = lane + k * TQK_WAVE;
        x[k] = 0.f;
        if (i >= dk) continue;
        float v = to_float(row[off + i]) + (bias ? to_float(bias[off + i]) : 0.f);
        if (rotate && i < rot_dim) {
            const bool first = style == 2 ? (i & 1) == 0 : i < half;
            const int partner = style == 2 ? (i ^ 1) : (first ? i + half : i - half);
            const int p = style == 2 ? i / 2 : (first ? i : i - half);
            const float y = to_float(row[off + partner]) + (bias ? to_float(bias[off + partner]) : 0.f);
            const float c = cos_table[(size_t)pos * half + p], s = sin_table[(size_t)pos * half + p];
            v = first ? v * c - y * s : v * c + y * s;
        }
        x[k] = v;
        ss = fmaf(v, v, ss);
    }
    const float inv = normed ? 1.f / sqrtf(wave_sum(ss) / (float)dk + eps) : 1.f;
    TA* dst = kind == 0 ? q_out + ((size_t)t * n_heads + head) * dk
                        : keys + (((size_t)page * n_kv_heads + (head - n_heads)) * TQK_PAGE + pos % TQK_PAGE) * dk;
#pragma unroll
    for (int k = 0; k < AM_MAX_D / TQK_WAVE; ++k) {
        const int i = lane + k * TQK_WAVE;
        if (i < dk) dst[i] = from_float<TA>(x[k] * inv);
    }
}

// Steps of many tokens in bfloat16, head sizes multiples of 8, in two launches.  Queries and keys: a wave per head as above, a lane
// takes VEC neighbouring elements in one load and one store (2 for heads up to 128, else 4); turned in pairs, an element's partner
// is in the same lane.  Values: the lanes along the tokens, as mixed_values_store_vec_kernel below has them.
template <typename TB, int VEC>
__global__ __launch_bounds__(AM_WAVES * TQK_WAVE)
void rope_norm_qk_vec_kernel(const bf16_t* __restrict__ qkv, const TB* __restrict__ bias, const float* __restrict__ cos_table,
                             const float* __restrict__ sin_table, int rot_dim, int style, int max_positions, int normed, float eps,
                             const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table,
                             int table_width, bf16_t* __restrict__ keys, bf16_t* __restrict__ q_out, int n_heads, int n_kv_heads, int dk, int dv,
                             int write_kv) {
    const int t = blockIdx.x;
    const int head = blockIdx.y * AM_WAVES + threadIdx.x / TQK_WAVE;
    const int lane = threadIdx.x % TQK_WAVE;
    if (head >= n_heads + (write_kv ? n_kv_heads : 0)) return;
    const int pos = tok_pos[t];
    const bool is_key = head >= n_heads;
    const size_t total = (size_t)(n_heads + n_kv_heads) * dk + (size_t)n_kv_heads * dv;
    const bf16_t* row = qkv + (size_t)t * total;
    int page = -1;
    if (is_key) {
        page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
        if (page < 0) return;                          // the host never lets this happen
    }
    const size_t off = (size_t)head * dk;
    const int half = rot_dim / 2;
    const bool rotate = rot_dim > 0 && style != 0 && pos < max_positions;
    const int i0 = lane * VEC;
    float x[VEC];
    float ss = 0.f;
    if (i0 < dk) {
        float raw[VEC];
        if (VEC == 2) {
            const uint32_t u = *reinterpret_cast<const uint32_t*>(row + off + i0);
            raw[0] = __uint_as_float(u << 16); raw[1] = __uint_as_float(u & 0xffff0000u);
        } else {
            const uint2 u = *reinterpret_cast<const uint2*>(row + off + i0);
            raw[0] = __uint_as_float(u.x << 16); raw[1] = __uint_as_float(u.x & 0xffff0000u);
            raw[VEC - 2] = __uint_as_float(u.y << 16); raw[VEC - 1] = __uint_as_float(u.y & 0xffff0000u);
        }
        if (bias) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) raw[j] += to_float(bias[off + i0 + j]);
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const int i = i0 + j;
            float v = raw[j];
            if (rotate && i < rot_dim) {
                bool first;
                float y;
                int p;
                if (style == 2) {
                    first = (j & 1) == 0; y = raw[j ^ 1]; p = i / 2;
                } else {
                    first = i < half;
                    const int partner = first ? i + half : i - half;
                    y = to_float(row[off + partner]) + (bias ? to_float(bias[off + partner]) : 0.f);
                    p = first ? i : i - half;
                }
                const float c = cos_table[(size_t)pos * half + p], sn = sin_table[(size_t)pos * half + p];
                v = first ? v * c - y * sn : v * c + y * sn;
            }
            x[j] = v;
            ss = fmaf(v, v, ss);
        }
    }
    const float inv = normed ? 1.f / sqrtf(wave_sum(ss) / (float)dk + eps) : 1.f;
    if (i0 >= dk) return;
    bf16_t* dst = !is_key ? q_out + ((size_t)t * n_heads + head) * dk
                          : keys + (((size_t)page * n_kv_heads + (head - n_heads)) * TQK_PAGE + pos % TQK_PAGE) * dk;
    uint32_t packed[VEC / 2];
#pragma unroll
    for (int j = 0; j < VEC / 2; ++j)
        packed[j] = (uint32_t)float_to_bf16_bits(x[2 * j] * inv) | ((uint32_t)float_to_bf16_bits(x[2 * j + 1] * inv) << 16);
    if (VEC == 2) *reinterpret_cast<uint32_t*>(dst + i0) = packed[0];
    else *reinterpret_cast<uint2*>(dst + i0) = make_uint2(packed[0], packed[VEC / 2 - 1]);
}

template <typename TB>
__global__ __launch_bounds__(256)
void biased_values_store_vec_kernel(const bf16_t* __restrict__ qkv, const TB* __restrict__ bias, const int32_t* __restrict__ tok_seq,
                                    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table, int table_width,
                                    bf16_t* __restrict__ values, int n_tokens, int n_heads, int n_kv_heads, int dk, int dv) {
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE, n_waves = blockDim.x / TQK_WAVE;
    const int t = (blockIdx.x / n_kv_heads) * TQK_WAVE + lane, g = blockIdx.x % n_kv_heads;
    if (t >= n_tokens) return;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
    if (page < 0) return;                               // the host never lets this happen
    bf16_t* dst = values + ((size_t)page * n_kv_heads + g) * TQK_PAGE * dv + value_place(pos % TQK_PAGE);
    const size_t total = (size_t)(n_heads + n_kv_heads) * dk + (size_t)n_kv_heads * dv;
    const size_t off = (size_t)(n_heads + n_kv_heads) * dk + (size_t)g * dv;
    const bf16_t* src = qkv + (size_t)t * total + off;
    for (int c = wave * 8; c < dv; c += n_waves * 8) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src + c);
        const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float lo = __uint_as_float(u[j] << 16), hi = __uint_as_float(u[j] & 0xffff0000u);
            if (bias) { lo += to_float(bias[off + c + 2 * j]); hi += to_float(bias[off + c + 2 * j + 1]); }
            dst[(size_t)(c + 2 * j) * TQK_PAGE].bits = float_to_bf16_bits(lo);
            dst[(size_t)(c + 2 * j + 1) * TQK_PAGE].bits = float_to_bf16_bits(hi);
        }
    }
}

// The same for steps of many tokens in bfloat16 (head sizes multiples of 8, half the rotated elements too), in two launches.
// Queries and keys: a block per token, a thread per 8 neighbouring elements (16 bytes a load and a store); the sums of squares of a
// head's pieces meet in LDS; the piece a rotated one turns with is read once more (it is in the caches).
template <typename TW>
__global__ __launch_bounds__(256)
void normed_rope_qk_vec_kernel(const bf16_t* __restrict__ qkv, const TW* __restrict__ q_norm_w, const TW* __restrict__ k_norm_w, float eps,
                               const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot_dim, int max_positions,
                               const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table,
                               int table_width, bf16_t* __restrict__ keys, bf16_t* __restrict__ q_out, int n_heads, int n_kv_heads, int dk, int dv,
                               int write_kv) {
    extern __shared__ float piece_ss[];
    const int t = blockIdx.x;
    const int per_head = dk / 8, n_pieces = (n_heads + (write_kv ? n_kv_heads : 0)) * per_head;
    const size_t total = (size_t)(n_heads + n_kv_heads) * dk + (size_t)n_kv_heads * dv;
    const bf16_t* row = qkv + (size_t)t * total;
    auto load8 = [&](const bf16_t* p, float* v) {
        const uint4 raw = *reinterpret_cast<const uint4*>(p);
        const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[2 * j] = __uint_as_float(u[j] << 16); v[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
    };
    const bool normed = q_norm_w != nullptr;
    if (normed) {
        for (int c = threadIdx.x; c < n_pieces; c += blockDim.x) {
            float x[8], ss = 0.f;
            load8(row + (size_t)c * 8, x);
#pragma unroll
            for (int j = 0; j < 8; ++j) ss = fmaf(x[j], x[j], ss);
            piece_ss[c] = ss;
        }
        __syncthreads();
    }
    const int pos = tok_pos[t];
    const int half = rot_dim / 2;
    const bool rotate = rot_dim > 0 && pos < max_positions;
    int page = -1;
    if (write_kv) page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
    for (int c = threadIdx.x; c < n_pieces; c += blockDim.x) {
        const int head = c / per_head, off = (c % per_head) * 8;
        const bool is_q = head < n_heads;
        if (!is_q && page < 0) continue;                // the host never lets this happen
        const TW* w = is_q ? q_norm_w : k_norm_w;
        float inv = 1.f;
        if (normed) {
            float ss = 0.f;
            for (int k = 0; k < per_head; ++k) ss += piece_ss[head * per_head + k];          // the same order for every piece of the head
            inv = 1.f / sqrtf(ss / (float)dk + eps);
        }
        float x[8];
        load8(row + (size_t)c * 8, x);
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] *= inv * (normed ? to_float(w[off + j]) : 1.f);
        if (rotate && off < rot_dim) {
            const bool first = off < half;
            const int other = first ? off + half : off - half, p = first ? off : off - half;
            float y[8];
            load8(row + (size_t)head * dk + other, y);
            // (half and p are multiples of 8: the eight angles of a piece are two aligned loads of 16 bytes from each table)
            const float4* ct = reinterpret_cast<const float4*>(cos_table + (size_t)pos * half + p);
            const float4* st = reinterpret_cast<const float4*>(sin_table + (size_t)pos * half + p);
            const float4 c0 = ct[0], c1 = ct[1], s0 = st[0], s1 = st[1];
            const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w}, sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float yn = y[j] * inv * (normed ? to_float(w[other + j]) : 1.f);
                x[j] = first ? x[j] * cs[j] - yn * sn[j] : x[j] * cs[j] + yn * sn[j];
            }
        }
        uint4 out;
        out.x = float_to_bf16_bits(x[0]) | ((uint32_t)float_to_bf16_bits(x[1]) << 16);
        out.y = float_to_bf16_bits(x[2]) | ((uint32_t)float_to_bf16_bits(x[3]) << 16);
        out.z = float_to_bf16_bits(x[4]) | ((uint32_t)float_to_bf16_bits(x[5]) << 16);
        out.w = float_to_bf16_bits(x[6]) | ((uint32_t)float_to_bf16_bits(x[7]) << 16);
        bf16_t* dst = is_q ? q_out + ((size_t)t * n_heads + head) * dk + off
                           : keys + (((size_t)page * n_kv_heads + (head - n_heads)) * TQK_PAGE + pos % TQK_PAGE) * dk + off;
        *reinterpret_cast<uint4*>(dst) = out;
    }
}

// Values: the cache keeps them transposed inside a page, so here the lanes run along the tokens (64 a block, one kv head, the waves
// taking pieces of 8 elements in turn): where the tokens are neighbours in a sequence, a wave's stores of one element fall into one row
// of 128 bytes.  Every lane finds its own page and place, so nothing depends on the tokens being neighbours.
template <typename TW>
__global__ __launch_bounds__(256)
void mixed_values_store_vec_kernel(const bf16_t* __restrict__ qkv, const TW* __restrict__ mix, const bf16_t* __restrict__ mix_with,
                                   bf16_t* __restrict__ mix_keep, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                   const int32_t* __restrict__ page_table, int table_width, bf16_t* __restrict__ values, int n_tokens, int n_heads,
                                   int n_kv_heads, int dk, int dv) {
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE, n_waves = blockDim.x / TQK_WAVE;
    const int t = (blockIdx.x / n_kv_heads) * TQK_WAVE + lane, g = blockIdx.x % n_kv_heads;
    if (t >= n_tokens) return;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
    if (page < 0) return;                               // the host never lets this happen
    bf16_t* dst = values + ((size_t)page * n_kv_heads + g) * TQK_PAGE * dv + value_place(pos % TQK_PAGE);
    const size_t total = (size_t)(n_heads + n_kv_heads) * dk + (size_t)n_kv_heads * dv;
    const bf16_t* src = qkv + (size_t)t * total + (size_t)(n_heads + n_kv_heads) * dk + (size_t)g * dv;
    const float lam = mix && mix_with ? to_float(mix[0]) : 0.f;
    for (int c = wave * 8; c < dv; c += n_waves * 8) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src + c);
        const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[2 * j] = __uint_as_float(u[j] << 16); v[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
        const size_t at = ((size_t)t * n_kv_heads + g) * dv + c;
        if (mix_with) {
            const uint4 mr = *reinterpret_cast<const uint4*>(mix_with + at);
            const uint32_t mu[4] = {mr.x, mr.y, mr.z, mr.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] = (1.f - lam) * v[2 * j] + lam * __uint_as_float(mu[j] << 16);
                v[2 * j + 1] = (1.f - lam) * v[2 * j + 1] + lam * __uint_as_float(mu[j] & 0xffff0000u);
            }
        }
        uint16_t bits[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) bits[j] = float_to_bf16_bits(v[j]);
        if (mix_keep) {
            uint4 out;
            out.x = bits[0] | ((uint32_t)bits[1] << 16);
            out.y = bits[2] | ((uint32_t)bits[3] << 16);
            out.z = bits[4] | ((uint32_t)bits[5] << 16);
            out.w = bits[6] | ((uint32_t)bits[7] << 16);
            *reinterpret_cast<uint4*>(mix_keep + at) = out;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[(size_t)(c + j) * TQK_PAGE].bits = bits[j];
    }
}

// ---- attention, a wave per (token, head) --------------------------------------------------------------
// Keys are taken a page at a time; lane j computes the score of key j of the page, the softmax runs online over the
// pages, then lane c accumulates output element c (+64, ...).  The order of operations for a query depends on its
// position alone.  Pages all of whose positions are hidden (between the kept first positions and the window) are
// passed over and may have been given back.
template <typename T, typename TS>
__global__ __launch_bounds__(AM_WAVES * TQK_WAVE)
void attention_masked_kernel(const T* __restrict__ q, const T* __restrict__ keys, const T* __restrict__ values,
                             const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                             const int32_t* __restrict__ page_table, int table_width, int window, int keep_first, float scale, float cap,
                             const TS* __restrict__ sink, T* __restrict__ out, int n_tokens, int n_heads, int n_kv_heads, int dk, int dv) {
    __shared__ float q_lds[AM_WAVES][AM_MAX_D];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int t = blockIdx.x * AM_WAVES + wave;
    const int head = blockIdx.y;
    const bool live = t < n_tokens;
    if (live) {
        const T* qv = q + ((size_t)t * n_heads + head) * dk;
        for (int i = lane; i < dk; i += TQK_WAVE) q_lds[wave][i] = to_float(qv[i]);
    }
    __syncthreads();
    if (!live) return;

    const int pos = tok_pos[t];
    const int32_t* pages = page_table + (size_t)tok_seq[t] * table_width;
    const int kvh = head / (n_heads / n_kv_heads);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int kept = window > 0 ? keep_first : 0;
    const float* qf = q_lds[wave];

    constexpr int NACC = AM_MAX_D / TQK_WAVE;
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    // the sink is a key of score sink_h without a value: the running maximum and sum start from it
    float m = sink ? to_float(sink[head]) : -INFINITY, l = sink ? 1.f : 0.f;

    for (int kb = 0; kb <= pos; kb += TQK_PAGE) {
        if (kb + TQK_PAGE <= lo && kb >= kept) continue;
        const int page = pages[kb / TQK_PAGE];
        const int j = kb + lane;
        const bool valid = j <= pos && (j >= lo || j < kept) && page >= 0;
        const size_t pg = (size_t)(page < 0 ? 0 : page) * n_kv_heads + kvh;
        float s = -INFINITY;
        if (valid) {
            const T* kr = keys + (pg * TQK_PAGE + lane) * dk;
            float dot = 0.f;
            for (int i = 0; i < dk; ++i) dot = fmaf(qf[i], to_float(kr[i]), dot);
            s = dot * scale;
            if (cap > 0.f) s = cap * tanhf(s / cap);
        }
        const float m_new = fmaxf(m, wave_max(s));     // finite: the page holds at least one visible key, or the sink came first
        const float p = valid ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);            // exp(-inf) = 0 on the first page
        l = l * alpha + wave_sum(p);
        m = m_new;
        const int n_keys = min(TQK_PAGE, pos - kb + 1);
        const T* vb = values + pg * TQK_PAGE * dv;
#pragma unroll
        for (int a = 0; a < NACC; ++a) {
            const int c = lane + a * TQK_WAVE;
            float sum = acc[a] * alpha;
            if (a * TQK_WAVE < dv) {
                for (int jj = 0; jj < n_keys; ++jj) {
                    const float pj = __shfl(p, jj, TQK_WAVE);
                    if (c < dv && pj != 0.f) sum = fmaf(pj, to_float(vb[(size_t)c * TQK_PAGE + value_place(jj)]), sum);
                }
            }
            acc[a] = sum;
        }
    }
    T* o = out + ((size_t)t * n_heads + head) * dv;
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const int c = lane + a * TQK_WAVE;
        if (c < dv) o[c] = from_float<T>(acc[a] / l);
    }
}

extern "C" int tqk_normed_rope_store(const void* qkv, int act_dtype, const void* q_norm_w, const void* k_norm_w, int w_dtype, float eps,
                                     const float* cos_table, const float* sin_table, int rot_dim, int max_positions, const void* mix,
                                     const void* mix_with, void* mix_keep, const int32_t* tok_seq, const int32_t* tok_pos,
                                     const int32_t* page_table, int table_width, void* keys, void* values, void* q_out, int n_tokens,
                                     int n_heads, int n_kv_heads, int key_dim, int value_dim, int write_kv, void* stream) {
    TQK_REQUIRE(qkv && tok_pos && q_out, "tqk_normed_rope_store: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && key_dim > 0 && value_dim > 0, "tqk_normed_rope_store: bad sizes");
    TQK_REQUIRE(rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= key_dim, "tqk_normed_rope_store: rot_dim %d must be even and <= key_dim %d", rot_dim, key_dim);
    TQK_REQUIRE(rot_dim == 0 || (cos_table && sin_table && max_positions > 0), "tqk_normed_rope_store: rotation without tables");
    TQK_REQUIRE(!write_kv || (tok_seq && page_table && keys && values && table_width > 0), "tqk_normed_rope_store: no cache to write to");
    TQK_REQUIRE(!mix_with || mix, "tqk_normed_rope_store: values to mix with, but no weight");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // steps of many tokens in bfloat16 whose sizes fall into pieces of 16 bytes: the two launches above
    const long long pieces = (long long)(n_heads + n_kv_heads) * key_dim / 8;
    if (act_dtype == TQK_BF16 && n_tokens > 64 && key_dim % 8 == 0 && value_dim % 8 == 0 && rot_dim % 16 == 0 && pieces <= 8192 &&
        (!q_norm_w) == (!k_norm_w)) {
        const size_t lds = (size_t)pieces * sizeof(float);
        const long long v_blocks = (long long)((n_tokens + TQK_WAVE - 1) / TQK_WAVE) * n_kv_heads;
        TQK_REQUIRE(v_blocks <= 0x7fffffff, "tqk_normed_rope_store: too many tokens");
#define TQK_NRV(TW) \
        normed_rope_qk_vec_kernel<TW><<<n_tokens, 256, lds, s>>>((const bf16_t*)qkv, (const TW*)q_norm_w, (const TW*)k_norm_w, eps, cos_table, sin_table, rot_dim, \
            max_positions, tok_seq, tok_pos, page_table, table_width, (bf16_t*)keys, (bf16_t*)q_out, n_heads, n_kv_heads, key_dim, value_dim, write_kv); \
        if (write_kv) mixed_values_store_vec_kernel<TW><<<(unsigned)v_blocks, 256, 0, s>>>((const bf16_t*)qkv, (const TW*)mix, (const bf16_t*)mix_with, \
            (bf16_t*)mix_keep, tok_seq, tok_pos, page_table, table_width, (bf16_t*)values, n_tokens, n_heads, n_kv_heads, key_dim, value_dim)
        if (w_dtype == TQK_F32) { TQK_NRV(float); } else if (w_dtype == TQK_BF16) { TQK_NRV(bf16_t); } else return tqk_fail("tqk_normed_rope_store: unknown dtype %d", w_dtype);
#undef TQK_NRV
        return tqk_check_launch("tqk_normed_rope_store");
    }
    dim3 grid(n_tokens, (n_heads + 2 * n_kv_heads + AM_WAVES - 1) / AM_WAVES);
#define TQK_NRS(TA, TW) \
    normed_rope_store_kernel<TA, TW><<<grid, AM_WAVES * TQK_WAVE, 0, s>>>((const TA*)qkv, (const TW*)q_norm_w, (const TW*)k_norm_w, eps, cos_table, sin_table, \
        rot_dim, max_positions, (const TW*)mix, (const TA*)mix_with, (TA*)mix_keep, tok_seq, tok_pos, page_table, table_width, (TA*)keys, (TA*)values, \
        (TA*)q_out, n_heads, n_kv_heads, key_dim, value_dim, write_kv)
    if (act_dtype == TQK_F32 && w_dtype == TQK_F32) TQK_NRS(float, float);
    else if (act_dtype == TQK_F32 && w_dtype == TQK_BF16) TQK_NRS(float, bf16_t);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_F32) TQK_NRS(bf16_t, float);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_BF16) TQK_NRS(bf16_t, bf16_t);
    else return tqk_fail("tqk_normed_rope_store: unknown dtypes %d, %d", act_dtype, w_dtype);
#undef TQK_NRS
    return tqk_check_launch("tqk_normed_rope_store");
}

extern "C" int tqk_rope_norm_store(const void* qkv, int act_dtype, const void* bias, int bias_dtype, const float* cos_table, const float* sin_table,
                                   int rot_dim, int style, int max_positions, int normed, float eps, const int32_t* tok_seq, const int32_t* tok_pos,
                                   const int32_t* page_table, int table_width, void* keys, void* values, void* q_out, int n_tokens, int n_heads,
                                   int n_kv_heads, int key_dim, int value_dim, int write_kv, void* stream) {
    TQK_REQUIRE(qkv && tok_pos && q_out, "tqk_rope_norm_store: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && key_dim > 0 && value_dim > 0, "tqk_rope_norm_store: bad sizes");
    TQK_REQUIRE(key_dim <= AM_MAX_D, "tqk_rope_norm_store: heads of %d values, the kernel takes up to %d", key_dim, AM_MAX_D);
    TQK_REQUIRE(style >= 0 && style <= 2, "tqk_rope_norm_store: unknown rotation style %d", style);
    TQK_REQUIRE(rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= key_dim, "tqk_rope_norm_store: rot_dim %d must be even and <= key_dim %d", rot_dim, key_dim);
    TQK_REQUIRE(rot_dim == 0 || style == 0 || (cos_table && sin_table && max_positions > 0), "tqk_rope_norm_store: rotation without tables");
    TQK_REQUIRE(!write_kv || (tok_seq && page_table && keys && values && table_width > 0), "tqk_rope_norm_store: no cache to write to");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == TQK_BF16 && n_tokens > 64 && key_dim % 8 == 0 && value_dim % 8 == 0 && (!bias || bias_dtype == TQK_BF16 || bias_dtype == TQK_F32) &&
        (((uintptr_t)qkv | (uintptr_t)keys | (uintptr_t)q_out) & 15) == 0) {
        dim3 qk_grid(n_tokens, (n_heads + (write_kv ? n_kv_heads : 0) + AM_WAVES - 1) / AM_WAVES);
        const long long v_blocks = (long long)((n_tokens + TQK_WAVE - 1) / TQK_WAVE) * n_kv_heads;
        TQK_REQUIRE(v_blocks <= 0x7fffffff, "tqk_rope_norm_store: too many tokens");
#define TQK_RNV(TB, VEC) \
        rope_norm_qk_vec_kernel<TB, VEC><<<qk_grid, AM_WAVES * TQK_WAVE, 0, s>>>((const bf16_t*)qkv, (const TB*)bias, cos_table, sin_table, rot_dim, style, \
            max_positions, normed, eps, tok_seq, tok_pos, page_table, table_width, (bf16_t*)keys, (bf16_t*)q_out, n_heads, n_kv_heads, key_dim, value_dim, write_kv)
#define TQK_RNV_ALL(TB) do { if (key_dim <= 128) TQK_RNV(TB, 2); else TQK_RNV(TB, 4); \
        if (write_kv) biased_values_store_vec_kernel<TB><<<(unsigned)v_blocks, 256, 0, s>>>((const bf16_t*)qkv, (const TB*)bias, tok_seq, tok_pos, page_table, \
            table_width, (bf16_t*)values, n_tokens, n_heads, n_kv_heads, key_dim, value_dim); } while (0)
        if (bias && bias_dtype == TQK_F32) TQK_RNV_ALL(float); else TQK_RNV_ALL(bf16_t);
#undef TQK_RNV_ALL
#undef TQK_RNV
        return tqk_check_launch("tqk_rope_norm_store");
    }
    dim3 grid(n_tokens, (n_heads + 2 * n_kv_heads + AM_WAVES - 1) / AM_WAVES);
#define TQK_RNS(TA, TB) \
    rope_norm_store_kernel<TA, TB><<<grid, AM_WAVES * TQK_WAVE, 0, s>>>((const TA*)qkv, (const TB*)bias, cos_table, sin_table, rot_dim, style, max_positions, \
        normed, eps, tok_seq, tok_pos, page_table, table_width, (TA*)keys, (TA*)values, (TA*)q_out, n_heads, n_kv_heads, key_dim, value_dim, write_kv)
    if (act_dtype == TQK_F32 && (!bias || bias_dtype == TQK_F32)) TQK_RNS(float, float);
    else if (act_dtype == TQK_F32 && bias_dtype == TQK_BF16) TQK_RNS(float, bf16_t);
    else if (act_dtype == TQK_BF16 && (!bias || bias_dtype == TQK_BF16)) TQK_RNS(bf16_t, bf16_t);
    else if (act_dtype == TQK_BF16 && bias_dtype == TQK_F32) TQK_RNS(bf16_t, float);
    else return tqk_fail("tqk_rope_norm_store: unknown dtypes %d, %d", act_dtype, bias_dtype);
#undef TQK_RNS
    return tqk_check_launch("tqk_rope_norm_store");
}

extern "C" int tqk_attention_masked_max_dim(void) { return AM_MAX_D; }

extern "C" int tqk_attention_masked(const void* q, const void* keys, const void* values, int act_dtype, const int32_t* tok_seq,
                                    const int32_t* tok_pos, const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window,
                                    int keep_first, float scale, float cap, const void* sink, int sink_dtype, void* out, int n_tokens,
                                    int n_heads, int n_kv_heads, int key_dim, int value_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_seq && tok_pos && page_table && out, "tqk_attention_masked: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && key_dim > 0 && value_dim > 0, "tqk_attention_masked: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention_masked: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(key_dim <= AM_MAX_D && value_dim <= AM_MAX_D, "tqk_attention_masked: head sizes %d and %d, the kernel takes up to %d", key_dim, value_dim, AM_MAX_D);
    TQK_REQUIRE(n_heads <= 65535, "tqk_attention_masked: too many heads for the grid");
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0, "tqk_attention_masked: empty page table");
    TQK_REQUIRE(window >= 0 && keep_first >= 0 && cap >= 0.f, "tqk_attention_masked: negative window, kept positions or cap");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((n_tokens + AM_WAVES - 1) / AM_WAVES, n_heads);
#define TQK_AM(T, TS) \
    attention_masked_kernel<T, TS><<<grid, AM_WAVES * TQK_WAVE, 0, s>>>((const T*)q, (const T*)keys, (const T*)values, tok_seq, tok_pos, page_table, \
        table_width, window, keep_first, scale, cap, (const TS*)sink, (T*)out, n_tokens, n_heads, n_kv_heads, key_dim, value_dim)
    if (act_dtype == TQK_F32 && (!sink || sink_dtype == TQK_F32)) TQK_AM(float, float);
    else if (act_dtype == TQK_F32 && sink_dtype == TQK_BF16) TQK_AM(float, bf16_t);
    else if (act_dtype == TQK_BF16 && (!sink || sink_dtype == TQK_BF16)) TQK_AM(bf16_t, bf16_t);
    else if (act_dtype == TQK_BF16 && sink_dtype == TQK_F32) TQK_AM(bf16_t, float);
    else return tqk_fail("tqk_attention_masked: unknown dtypes %d, %d", act_dtype, sink_dtype);
#undef TQK_AM
    return tqk_check_launch("tqk_attention_masked");
}
