// A feed-forward of routed experts: the router, the grouping of a step's (token, expert) pairs by
// expert, the experts' products over the grouped rows, and the weighted sum.
//
//   route     z = W_r x in float32, s = softmax(z) over all experts, the `top` largest (the lower index wins
//             a tie); weight = s * scale, not renormalised.  One wave per token.  Mode bit 1 renormalises over the chosen;
//             mode bit 2 makes every expert's score sigmoid(z) on its own instead of the softmax.
//   scale     rows[pair_pos[p]] = weight[p] * x[p / top] (for experts whose input, not output, carries the weight), and unit[p] = 1
//   group     pair p = (token p / top, choice p % top) gets a row of its own among its expert's rows:
//             pair_pos[p]; sorted_tok[row] names the row's token.  The rows of an expert are cut into tiles of
//             tile_m rows; the tile list (expert, first row, rows) and its length stay on the device, so the
//             launches that follow have the same shape whatever the router chose.
//   product   for each tile, rows x (gathered through sorted_tok, or as they lie) times the tile's expert's
//             weight: plain, or gate and up with the gate applied.  Blocks beyond the list's length exit.
//   combine   out[t] = sum_k weight[t, k] * y[pair_pos[t, k]] (+ what a shared expert gave), in float32.
//
// A row's sums never depend on which rows share its tile, nor on the order the pairs were given rows in.
#include "common.h"
#include "tq_kernels.h"

#define MOE_MAX_EXPERTS 512
#define MOE_ROUTE_WAVES 8
#define MOE_TM 32               // rows of a tile
#define MOE_TN 64               // features of a block
#define MOE_TK 16               // k per stage

// ---- route -----------------------------------------------------------------------------------
// A block per token: its waves share the experts out for the logits (each a dot product over the lanes, several loads
// under way at once, added up in a fixed order), then the first wave takes the softmax and the largest.
template <typename TA, typename TW>
__global__ __launch_bounds__(MOE_ROUTE_WAVES * TQK_WAVE)
void moe_route_kernel(const TA* __restrict__ x, const TW* __restrict__ w, int n_experts, int hidden, int top, float scale, int mode,
                      int32_t* __restrict__ idx, float* __restrict__ weight, const TW* __restrict__ gate_w, float* __restrict__ gate_out) {
    const int renormalize = mode & 1, sigmoid_scores = mode & 2;
    __shared__ float z[MOE_MAX_EXPERTS];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int t = blockIdx.x;
    const TA* xr = x + (size_t)t * hidden;
    // one row more where a gate is given: sigmoid(x . gate_w) per token, which rides along with the experts' dot products
    for (int e = wave; e < n_experts + (gate_w ? 1 : 0); e += MOE_ROUTE_WAVES) {
        const TW* wr = e < n_experts ? w + (size_t)e * hidden : gate_w;
        float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
        int i = lane;
        if (sizeof(TA) == 2 && sizeof(TW) == 2 && hidden % 8 == 0) {
            // bfloat16 rows whose length is a multiple of 8: 16 bytes a lane and load, in the same order of additions for
            // every token
            float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int c = lane * 8; c < hidden; c += TQK_WAVE * 8) {
                const uint4 xv = *reinterpret_cast<const uint4*>(xr + c), wv = *reinterpret_cast<const uint4*>(wr + c);
                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    d[2 * k] = fmaf(__uint_as_float(xw[k] << 16), __uint_as_float(ww[k] << 16), d[2 * k]);
                    d[2 * k + 1] = fmaf(__uint_as_float(xw[k] & 0xffff0000u), __uint_as_float(ww[k] & 0xffff0000u), d[2 * k + 1]);
                }
            }
            d0 = (d[0] + d[1]) + (d[2] + d[3]);
            d1 = (d[4] + d[5]) + (d[6] + d[7]);
            i = hidden;
        }
        for (; i + 3 * TQK_WAVE < hidden; i += 4 * TQK_WAVE) {
            d0 = fmaf(to_float(xr[i]), to_float(wr[i]), d0);
            d1 = fmaf(to_float(xr[i + TQK_WAVE]), to_float(wr[i + TQK_WAVE]), d1);
            d2 = fmaf(to_float(xr[i + 2 * TQK_WAVE]), to_float(wr[i + 2 * TQK_WAVE]), d2);
            d3 = fmaf(to_float(xr[i + 3 * TQK_WAVE]), to_float(wr[i + 3 * TQK_WAVE]), d3);
        }
        for (; i < hidden; i += TQK_WAVE) d0 = fmaf(to_float(xr[i]), to_float(wr[i]), d0);
        const float dot = wave_sum((d0 + d1) + (d2 + d3));
        if (lane == 0) {
            if (e < n_experts) z[e] = dot;
            else gate_out[t] = 1.f / (1.f + expf(-dot));
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float m = -INFINITY;
    for (int e = lane; e < n_experts; e += TQK_WAVE) m = fmaxf(m, z[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < n_experts; e += TQK_WAVE) sum += expf(z[e] - m);
    sum = wave_sum(sum);
    // what the lane's experts still offer; a chosen one is struck out in the registers of the lane that holds it
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int best_e = 0x7fffffff;
        for (int e = lane; e < n_experts; e += TQK_WAVE) {
            const float v = z[e];
            if (v > best) { best = v; best_e = e; }         // increasing e: the lower index stays on a tie
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, TQK_WAVE);
            const int oe = __shfl_xor(best_e, o, TQK_WAVE);
            if (ov > best || (ov == best && oe < best_e)) { best = ov; best_e = oe; }
        }
        if (lane == best_e % TQK_WAVE) z[best_e] = -INFINITY;       // the lane that reads this expert writes it: no other sees it
        if (lane == 0) {
            idx[(size_t)t * top + k] = best_e;
            weight[(size_t)t * top + k] = (sigmoid_scores ? 1.f / (1.f + expf(-best)) : expf(best - m) / sum) * scale;
        }
    }
    if (!renormalize) return;
    // the softmax over the chosen logits alone: the chosen scores divided by their sum, added up in the order they were chosen
    if (lane == 0) {
        float chosen = 0.f;
        for (int k = 0; k < top; ++k) chosen += weight[(size_t)t * top + k];
        for (int k = 0; k < top; ++k) weight[(size_t)t * top + k] /= chosen;
    }
}

// ---- group -----------------------------------------------------------------------------------
__global__ __launch_bounds__(1024)
void moe_group_kernel(const int32_t* __restrict__ idx, int n_pairs, int top, int n_experts, int tile_m, int32_t* __restrict__ pair_pos,
                      int32_t* __restrict__ sorted_tok, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
                      int32_t* __restrict__ tile_rows, int32_t* __restrict__ n_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS], offset[MOE_MAX_EXPERTS], tile_base[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) pair_pos[p] = atomicAdd(&count[idx[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int rows = 0, tiles = 0;
        for (int e = 0; e < n_experts; ++e) {
            offset[e] = rows;
            tile_base[e] = tiles;
            rows += count[e];
            tiles += (count[e] + tile_m - 1) / tile_m;
        }
        *n_tiles = tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        const int n = count[e];
        for (int i = 0, tile = tile_base[e]; i < n; i += tile_m, ++tile) {
            tile_expert[tile] = e;
            tile_row0[tile] = offset[e] + i;
            tile_rows[tile] = min(tile_m, n - i);
        }
    }
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int row = offset[idx[p]] + pair_pos[p];
        pair_pos[p] = row;
        sorted_tok[row] = p / top;
    }
}

// ---- product ---------------------------------------------------------------------------------
// 32 rows x 64 features per block, 2 x 4 per thread, float32 fused multiply-adds in increasing k.
template <typename TX, typename TW, typename TY, bool GATED>
__global__ __launch_bounds__(256)
void moe_product_kernel(const TX* __restrict__ x, const int32_t* __restrict__ x_rows, const TW* __restrict__ w, long long expert_stride,
                        TY* __restrict__ y, int N, int K, int gate, float limit, float alpha, const int32_t* __restrict__ tile_expert,
                        const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ tile_rows, const int32_t* __restrict__ n_tiles) {
    const int tile = blockIdx.y;
    if (tile >= *n_tiles) return;
    __shared__ float xs[MOE_TK][MOE_TM + 2];
    __shared__ float ws[GATED ? 2 : 1][MOE_TK][MOE_TN + 4];
    const int expert = tile_expert[tile], row0 = tile_row0[tile], n_rows = tile_rows[tile];
    const int n0 = blockIdx.x * MOE_TN;
    const TW* we = w + (size_t)expert * expert_stride;
    const int tid = threadIdx.x, tm = tid / 16, tn = tid % 16;
    float acc[GATED ? 2 : 1][2][4];
#pragma unroll
    for (int g = 0; g < (GATED ? 2 : 1); ++g)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[g][i][j] = 0.f;
    // the two x elements and the four weight elements a thread brings in per stage
    const int xr0 = tid / MOE_TK, xk = tid % MOE_TK;                // rows xr0 and xr0 + 16
    long long xsrc[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int r = xr0 + 16 * e;
        xsrc[e] = r < n_rows ? (long long)(x_rows ? x_rows[row0 + r] : row0 + r) * K : -1;
    }
    for (int k0 = 0; k0 < K; k0 += MOE_TK) {
#pragma unroll
        for (int e = 0; e < 2; ++e) xs[xk][xr0 + 16 * e] = (xsrc[e] >= 0 && k0 + xk < K) ? to_float(x[xsrc[e] + k0 + xk]) : 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int i = tid + e * 256, r = i / MOE_TK, kk = i % MOE_TK;
            const bool in = n0 + r < N && k0 + kk < K;
            ws[0][kk][r] = in ? to_float(we[(size_t)(n0 + r) * K + k0 + kk]) : 0.f;
            if (GATED) ws[GATED ? 1 : 0][kk][r] = in ? to_float(we[(size_t)(N + n0 + r) * K + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < MOE_TK; ++kk) {
            const float a0 = xs[kk][tm * 2], a1 = xs[kk][tm * 2 + 1];
#pragma unroll
            for (int g = 0; g < (GATED ? 2 : 1); ++g)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float b = ws[g][kk][tn * 4 + j];
                    acc[g][0][j] = fmaf(a0, b, acc[g][0][j]);
                    acc[g][1][j] = fmaf(a1, b, acc[g][1][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = tm * 2 + i;
        if (r >= n_rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn * 4 + j;
            if (n >= N) continue;
            float v = acc[0][i][j];
            if (GATED) {
                // gate and up are rounded as stored products would be, then the gate in float32
                const float g = to_float(from_float<TY>(v)), u = to_float(from_float<TY>(acc[GATED ? 1 : 0][i][j]));
                v = gate_value(gate, limit, alpha, g, u);
            } else if (gate >= 0) {
                v = act_value(gate, limit, alpha, to_float(from_float<TY>(v)));
            }
            y[(size_t)(row0 + r) * N + n] = from_float<TY>(v);
        }
    }
}

// ---- combine ---------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256)
void moe_combine_kernel(const TA* __restrict__ y, const int32_t* __restrict__ pair_pos, const float* __restrict__ weight, int top,
                        const TA* __restrict__ shared, const float* __restrict__ shared_scale, TA* __restrict__ out, int hidden) {
    // the token's rows and weights once, side by side, not one load after the other in front of every element
    __shared__ int32_t row[MOE_MAX_EXPERTS];
    __shared__ float wt[MOE_MAX_EXPERTS];
    const int t = blockIdx.x;
    for (int k = threadIdx.x; k < top; k += blockDim.x) {
        row[k] = pair_pos[(size_t)t * top + k];
        wt[k] = weight[(size_t)t * top + k];
    }
    __syncthreads();
    const float ss = shared && shared_scale ? shared_scale[t] : 1.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = 0.f;
#pragma unroll 4
        for (int k = 0; k < top; ++k) v = fmaf(wt[k], to_float(y[(size_t)row[k] * hidden + i]), v);
        if (shared) v = fmaf(ss, to_float(shared[(size_t)t * hidden + i]), v);
        out[(size_t)t * hidden + i] = from_float<TA>(v);
    }
}

// ---- scale -----------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256)
void moe_scale_rows_kernel(const TA* __restrict__ x, const int32_t* __restrict__ pair_pos, const float* __restrict__ weight, int top,
                           TA* __restrict__ rows, float* __restrict__ unit, int hidden) {
    const size_t p = blockIdx.x;
    const float w = weight[p];
    const TA* src = x + (p / top) * hidden;
    TA* dst = rows + (size_t)pair_pos[p] * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = from_float<TA>(w * to_float(src[i]));
    if (threadIdx.x == 0) unit[p] = 1.f;
}

// ---- entry points ----------------------------------------------------------------------------
extern "C" int tqk_moe_scale_rows(const void* x, int act_dtype, const int32_t* pair_pos, const float* weight, int top, void* rows, float* unit,
                                  int n_tokens, int hidden, void* stream) {
    TQK_REQUIRE(x && pair_pos && weight && rows && unit, "tqk_moe_scale_rows: null pointer");
    TQK_REQUIRE(top > 0 && hidden > 0 && n_tokens >= 0 && (long long)n_tokens * top <= 0x7fffffff, "tqk_moe_scale_rows: bad sizes");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned pairs = (unsigned)(n_tokens * top);
    if (act_dtype == TQK_F32) moe_scale_rows_kernel<float><<<pairs, 256, 0, s>>>((const float*)x, pair_pos, weight, top, (float*)rows, unit, hidden);
    else if (act_dtype == TQK_BF16) moe_scale_rows_kernel<bf16_t><<<pairs, 256, 0, s>>>((const bf16_t*)x, pair_pos, weight, top, (bf16_t*)rows, unit, hidden);
    else return tqk_fail("tqk_moe_scale_rows: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_moe_scale_rows");
}

extern "C" int tqk_moe_max_experts(void) { return MOE_MAX_EXPERTS; }
extern "C" int tqk_moe_tile_rows(void) { return MOE_TM; }
extern "C" int tqk_moe_max_tiles(int n_pairs, int n_experts, int tile_m) { return (n_pairs + tile_m - 1) / tile_m + n_experts; }

extern "C" int tqk_moe_route(const void* x, int act_dtype, const void* w_router, int w_dtype, int n_experts, int hidden, int top, float scale,
                             int mode, int32_t* idx, float* weight, const void* gate_w, float* gate_out, int n_tokens, void* stream) {
    TQK_REQUIRE(x && w_router && idx && weight, "tqk_moe_route: null pointer");
    TQK_REQUIRE(n_experts > 0 && n_experts <= MOE_MAX_EXPERTS, "tqk_moe_route: %d experts, the kernel takes 1 to %d", n_experts, MOE_MAX_EXPERTS);
    TQK_REQUIRE(top > 0 && top <= n_experts && hidden > 0 && n_tokens >= 0, "tqk_moe_route: bad sizes (top %d of %d experts)", top, n_experts);
    TQK_REQUIRE(!gate_w || gate_out, "tqk_moe_route: a gate without a place for its values");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TQK_ROUTE(TA, TW) \
    moe_route_kernel<TA, TW><<<n_tokens, MOE_ROUTE_WAVES * TQK_WAVE, 0, s>>>((const TA*)x, (const TW*)w_router, n_experts, hidden, top, scale, mode, idx, weight, (const TW*)gate_w, gate_out)
    if (act_dtype == TQK_F32 && w_dtype == TQK_F32) TQK_ROUTE(float, float);
    else if (act_dtype == TQK_F32 && w_dtype == TQK_BF16) TQK_ROUTE(float, bf16_t);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_F32) TQK_ROUTE(bf16_t, float);
    else if (act_dtype == TQK_BF16 && w_dtype == TQK_BF16) TQK_ROUTE(bf16_t, bf16_t);
    else return tqk_fail("tqk_moe_route: unknown dtypes %d, %d", act_dtype, w_dtype);
#undef TQK_ROUTE
    return tqk_check_launch("tqk_moe_route");
}

extern "C" int tqk_moe_group(const int32_t* idx, int n_tokens, int top, int n_experts, int tile_m, int32_t* pair_pos, int32_t* sorted_tok,
                             int32_t* tile_expert, int32_t* tile_row0, int32_t* tile_rows, int32_t* n_tiles, void* stream) {
    TQK_REQUIRE(idx && pair_pos && sorted_tok && tile_expert && tile_row0 && tile_rows && n_tiles, "tqk_moe_group: null pointer");
    TQK_REQUIRE(n_experts > 0 && n_experts <= MOE_MAX_EXPERTS && top > 0 && n_tokens >= 0, "tqk_moe_group: bad sizes");
    TQK_REQUIRE((long long)n_tokens * top <= 0x7fffffff, "tqk_moe_group: too many pairs");
    TQK_REQUIRE(tile_m > 0, "tqk_moe_group: tiles of %d rows", tile_m);
    if (n_tokens == 0) return 0;
    moe_group_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(idx, n_tokens * top, top, n_experts, tile_m, pair_pos, sorted_tok, tile_expert, tile_row0,
                                                          tile_rows, n_tiles);
    return tqk_check_launch("tqk_moe_group");
}

template <typename TX, typename TW, typename TY>
static int launch_moe_product(const void* x, const int32_t* x_rows, const void* w, long long expert_stride, void* y, int N, int K, int gated,
                              int gate, float limit, float alpha, const int32_t* tile_expert, const int32_t* tile_row0,
                              const int32_t* tile_rows, const int32_t* n_tiles, int max_tiles, hipStream_t s) {
    dim3 grid((N + MOE_TN - 1) / MOE_TN, max_tiles);
    if (gated == 1)
        moe_product_kernel<TX, TW, TY, true><<<grid, 256, 0, s>>>((const TX*)x, x_rows, (const TW*)w, expert_stride, (TY*)y, N, K, gate, limit, alpha,
                                                                  tile_expert, tile_row0, tile_rows, n_tiles);
    else
        moe_product_kernel<TX, TW, TY, false><<<grid, 256, 0, s>>>((const TX*)x, x_rows, (const TW*)w, expert_stride, (TY*)y, N, K, gated == 2 ? gate : -1, limit, alpha,
                                                                   tile_expert, tile_row0, tile_rows, n_tiles);
    return tqk_check_launch("tqk_moe_product");
}

extern "C" int tqk_moe_product(const void* x, int act_dtype, const int32_t* x_rows, const void* w, int w_dtype, long long expert_stride, void* y,
                               int N, int K, int gated, int gate, float limit, float alpha, const int32_t* tile_expert,
                               const int32_t* tile_row0, const int32_t* tile_rows, const int32_t* n_tiles, int max_tiles, void* stream) {
    TQK_REQUIRE(x && w && y && tile_expert && tile_row0 && tile_rows && n_tiles, "tqk_moe_product: null pointer");
    TQK_REQUIRE(N > 0 && K > 0 && max_tiles >= 0 && max_tiles <= 65535, "tqk_moe_product: bad sizes (N %d, K %d, %d tiles)", N, K, max_tiles);
    TQK_REQUIRE(gated >= 0 && gated <= 2, "tqk_moe_product: gated must be 0 (plain), 1 (gate and up) or 2 (one product with its activation), got %d", gated);
    TQK_REQUIRE(!gated || (gate >= 0 && gate < TQK_GATE_KINDS), "tqk_moe_product: unknown gate %d", gate);
    TQK_REQUIRE(expert_stride >= (long long)(gated == 1 ? 2 : 1) * N * K, "tqk_moe_product: experts overlap");
    /* the tile lists must have been made for tiles of tqk_moe_tile_rows() rows */
    if (max_tiles == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TQK_MOE(TX, TW) \
    return launch_moe_product<TX, TW, TX>(x, x_rows, w, expert_stride, y, N, K, gated, gate, limit, alpha, tile_expert, tile_row0, tile_rows, n_tiles, max_tiles, s)
    if (act_dtype == TQK_F32 && w_dtype == TQK_F32) TQK_MOE(float, float);
    if (act_dtype == TQK_F32 && w_dtype == TQK_BF16) TQK_MOE(float, bf16_t);
    if (act_dtype == TQK_BF16 && w_dtype == TQK_F32) TQK_MOE(bf16_t, float);
    if (act_dtype == TQK_BF16 && w_dtype == TQK_BF16) TQK_MOE(bf16_t, bf16_t);
#undef TQK_MOE
    return tqk_fail("tqk_moe_product: unknown dtypes %d, %d", act_dtype, w_dtype);
}

extern "C" int tqk_moe_combine(const void* y, int act_dtype, const int32_t* pair_pos, const float* weight, int top, const void* shared,
                               const float* shared_scale, void* out, int n_tokens, int hidden, void* stream) {
    TQK_REQUIRE(y && pair_pos && weight && out, "tqk_moe_combine: null pointer");
    TQK_REQUIRE(top > 0 && top <= MOE_MAX_EXPERTS && hidden > 0 && n_tokens >= 0, "tqk_moe_combine: bad sizes");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == TQK_F32)
        moe_combine_kernel<float><<<n_tokens, 256, 0, s>>>((const float*)y, pair_pos, weight, top, (const float*)shared, shared_scale, (float*)out, hidden);
    else if (act_dtype == TQK_BF16)
        moe_combine_kernel<bf16_t><<<n_tokens, 256, 0, s>>>((const bf16_t*)y, pair_pos, weight, top, (const bf16_t*)shared, shared_scale, (bf16_t*)out, hidden);
    else return tqk_fail("tqk_moe_combine: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_moe_combine");
}
