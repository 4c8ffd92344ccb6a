// Softmax attention over a sliding window plus one pooled key and value for every block of `pool` positions that lies wholly in
// front of the window, with an optional sink in the denominator and values that are turned by their position on the way into the
// cache and turned back, by the query's position, on the way out.
//
// Position i sees the positions j with 0 <= i - j < window, and block b (positions b pool .. b pool + pool - 1) if
// b pool + pool - 1 <= i - window; a block's key and value are the means of its positions' as the cache holds them.
//
// The cache's pages (TQK_PAGE positions each) hold, per kv head, the page's positions' rows followed by `pooled_rows` rows for the
// blocks whose last position falls into the page: keys [kv heads][TQK_PAGE + pooled_rows][d], values [kv heads][TQK_PAGE +
// pooled_rows][dv].  Block b, whose last position is e = b pool + pool - 1, lies in page e / TQK_PAGE at row
// TQK_PAGE + b - (e / TQK_PAGE) TQK_PAGE / pool (integer divisions).
//
//   tqk_pooled_store      from the q/k/v product of the step's tokens: q and k heads divided by their root mean square and multiplied by
//                         a weight (optional), their first rot_dim elements turned by the position, values turned over all their
//                         elements (optional); q out, k and v into the pages
//   tqk_pool_blocks       the means of the blocks that the step completes
//   tqk_pooled_attention  a wave per (row, head): blocks first, then the window's positions, 64 at a time: a lane a key for the scores,
//                         a lane an output element (and every 64th after it) for the values; softmax in float32.  Heads of 8 n key
//                         elements and 2 n values: several waves per (row, head) and wider loads
#include "common.h"
#include "tq_kernels.h"

enum { PA_STYLE_NONE = 0, PA_STYLE_HALVES = 1, PA_STYLE_PAIRS = 2 };
#define PA_MAX_DIM 256

__device__ __forceinline__ int pa_pooled_row(int b, int pool) {
    const int e = b * pool + pool - 1, page = e / TQK_PAGE;
    return TQK_PAGE + b - (page * TQK_PAGE) / pool;
}

// element i of a head turned by the angle of (pos, i's pair): x the head's values through `get`
template <typename F>
__device__ __forceinline__ float pa_turned(F get, int i, int rot_dim, int style, const float* cos, const float* sin, int pos, float sign) {
    const float v = get(i);
    if (style == PA_STYLE_NONE || i >= rot_dim) return v;
    const int half = rot_dim / 2;
    bool first;
    int pi, ai;
    if (style == PA_STYLE_HALVES) { first = i < half; pi = first ? i + half : i - half; ai = first ? i : i - half; }
    else { first = !(i & 1); pi = i ^ 1; ai = i >> 1; }
    const float c = cos[(size_t)pos * half + ai], s = sign * sin[(size_t)pos * half + ai];
    const float p = get(pi);
    return first ? v * c - p * s : v * c + p * s;
}

// a wave per (token, head of q, k or v)
template <typename T>
__global__ __launch_bounds__(256)
void pooled_store_kernel(const T* __restrict__ qkv, const float* __restrict__ q_w, const float* __restrict__ k_w, int normed, float eps,
                         const float* __restrict__ cos, const float* __restrict__ sin, int rot_dim, int style, const float* __restrict__ vcos,
                         const float* __restrict__ vsin, int max_pos, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                         const int32_t* __restrict__ table, int width, T* __restrict__ keys, T* __restrict__ values, T* __restrict__ q_out,
                         long long n_items, int H, int G, int d, int dv, int page_rows) {
    const long long item = (long long)blockIdx.x * (256 / TQK_WAVE) + threadIdx.x / TQK_WAVE;
    if (item >= n_items) return;
    const int lane = threadIdx.x % TQK_WAVE;
    const int per_tok = H + 2 * G;
    const long long t = item / per_tok;
    const int slot = (int)(item % per_tok);
    const size_t row_len = (size_t)(H + G) * d + (size_t)G * dv;
    const int pos = min(tok_pos[t], max_pos - 1);
    const int page = table[(size_t)tok_seq[t] * width + tok_pos[t] / TQK_PAGE], in_page = tok_pos[t] % TQK_PAGE;
    if (slot < H + G) {
        const bool is_q = slot < H;
        const T* x = qkv + (size_t)t * row_len + (size_t)slot * d;
        const float* w = is_q ? q_w : k_w;
        float inv = 1.f;
        if (normed) {
            float ss = 0.f;
            for (int i = lane; i < d; i += TQK_WAVE) { const float v = to_float(x[i]); ss = fmaf(v, v, ss); }
            inv = 1.f / sqrtf(wave_sum(ss) / (float)d + eps);
        }
        auto get = [&](int i) { float v = to_float(x[i]); if (normed) { v *= inv; if (w) v *= w[i]; } return v; };
        T* dst = is_q ? q_out + ((size_t)t * H + slot) * d
                      : keys + (((size_t)page * G + (slot - H)) * page_rows + in_page) * d;
        for (int i = lane; i < d; i += TQK_WAVE) dst[i] = from_float<T>(pa_turned(get, i, rot_dim, style, cos, sin, pos, 1.f));
    } else {
        const int g = slot - H - G;
        const T* x = qkv + (size_t)t * row_len + (size_t)(H + G) * d + (size_t)g * dv;
        auto get = [&](int i) { return to_float(x[i]); };
        T* dst = values + (((size_t)page * G + g) * page_rows + in_page) * dv;
        for (int i = lane; i < dv; i += TQK_WAVE) dst[i] = from_float<T>(pa_turned(get, i, dv, vcos ? style : PA_STYLE_NONE, vcos, vsin, pos, 1.f));
    }
}

// grid (blocks a sequence may complete, kv heads, sequences); a thread an element of the key or of the value
template <typename T>
__global__ __launch_bounds__(256)
void pool_blocks_kernel(T* __restrict__ keys, T* __restrict__ values, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_new,
                        const int32_t* __restrict__ table, int width, int pool, int G, int d, int dv, int page_rows) {
    const int s = blockIdx.z, g = blockIdx.y;
    const int start = seq_start[s], end = start + seq_new[s];
    const int b = start / pool + blockIdx.x;
    if (b >= end / pool) return;
    const int e_last = b * pool + pool - 1;
    const int dst_page = table[(size_t)s * width + e_last / TQK_PAGE], dst_row = pa_pooled_row(b, pool);
    const float inv = 1.f / (float)pool;
    for (int e = threadIdx.x; e < d + dv; e += blockDim.x) {
        const bool is_k = e < d;
        const int i = is_k ? e : e - d, len = is_k ? d : dv;
        T* base = is_k ? keys : values;
        float sum = 0.f;
        for (int p = b * pool; p <= e_last; ++p) {
            const int page = table[(size_t)s * width + p / TQK_PAGE];
            sum += to_float(base[(((size_t)page * G + g) * page_rows + p % TQK_PAGE) * len + i]);
        }
        base[(((size_t)dst_page * G + g) * page_rows + dst_row) * len + i] = from_float<T>(sum * inv);
    }
}

template <typename T>
__global__ __launch_bounds__(256)
void pooled_attention_kernel(const T* __restrict__ q, const T* __restrict__ keys, const T* __restrict__ values, const int32_t* __restrict__ row_seq,
                             const int32_t* __restrict__ row_pos, const int32_t* __restrict__ table, int width, int window, int pool, float scale,
                             const float* __restrict__ sink, const float* __restrict__ vcos, const float* __restrict__ vsin, int style, int max_pos,
                             T* __restrict__ out, long long n_items, int H, int G, int d, int dv, int page_rows) {
    __shared__ float q_lds[256 / TQK_WAVE][PA_MAX_DIM];
    __shared__ float o_lds[256 / TQK_WAVE][PA_MAX_DIM];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const long long item = (long long)blockIdx.x * (256 / TQK_WAVE) + wave;
    if (item >= n_items) return;
    const long long r = item / H;
    const int h = (int)(item % H), g = h / (H / G);
    const int pos = row_pos[r];
    const int32_t* pages = table + (size_t)row_seq[r] * width;
    float* ql = q_lds[wave];
    for (int i = lane; i < d; i += TQK_WAVE) ql[i] = to_float(q[((size_t)r * H + h) * d + i]) * scale;
    const int lo = max(0, pos - window + 1);
    const int n_blocks = pos - window + 1 >= pool ? (pos - window + 1) / pool : 0;
    const int n_all = n_blocks + (pos - lo + 1);
    float m = -INFINITY, l = 0.f;
    float acc[PA_MAX_DIM / TQK_WAVE];
#pragma unroll
    for (int c = 0; c < PA_MAX_DIM / TQK_WAVE; ++c) acc[c] = 0.f;
    for (int n0 = 0; n0 < n_all; n0 += TQK_WAVE) {
        const int n = n0 + lane;
        long long row = -1;            // the item's row among all rows of the pages: (page * G + g) * page_rows + row in page
        if (n < n_all) {
            int page, in_page;
            if (n < n_blocks) { page = pages[(n * pool + pool - 1) / TQK_PAGE]; in_page = pa_pooled_row(n, pool); }
            else { const int j = lo + (n - n_blocks); page = pages[j / TQK_PAGE]; in_page = j % TQK_PAGE; }
            row = ((long long)page * G + g) * page_rows + in_page;
        }
        float s = -INFINITY;
        if (row >= 0) {
            const T* kr = keys + (size_t)row * d;
            float dot = 0.f;
            for (int i = 0; i < d; ++i) dot = fmaf(ql[i], to_float(kr[i]), dot);
            s = dot;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float corr = expf(m - m_new);          // m = -inf at first: 0
        const float p = row >= 0 ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int c = 0; c < PA_MAX_DIM / TQK_WAVE; ++c) acc[c] *= corr;
        const int n_here = min(TQK_WAVE, n_all - n0);
        for (int k = 0; k < n_here; ++k) {
            const float pk = __shfl(p, k, TQK_WAVE);
            const long long rk = __shfl(row, k, TQK_WAVE);
            const T* vr = values + (size_t)rk * dv;
#pragma unroll
            for (int c = 0; c < PA_MAX_DIM / TQK_WAVE; ++c) {
                const int i = c * TQK_WAVE + lane;
                if (i < dv) acc[c] = fmaf(pk, to_float(vr[i]), acc[c]);
            }
        }
    }
    if (sink) {
        const float sv = sink[h], m_new = fmaxf(m, sv);
        const float corr = expf(m - m_new);
        l = l * corr + expf(sv - m_new);
#pragma unroll
        for (int c = 0; c < PA_MAX_DIM / TQK_WAVE; ++c) acc[c] *= corr;
    }
    const float inv = 1.f / l;
    float* ol = o_lds[wave];
#pragma unroll
    for (int c = 0; c < PA_MAX_DIM / TQK_WAVE; ++c) {
        const int i = c * TQK_WAVE + lane;
        if (i < dv) ol[i] = acc[c] * inv;
    }
    // (a wave's lanes run together: what the lanes wrote above is there for all of them)
    __builtin_amdgcn_wave_barrier();
    auto get = [&](int i) { return ol[i]; };
    const int tpos = min(pos, max_pos - 1);
    for (int i = lane; i < dv; i += TQK_WAVE)
        out[((size_t)r * H + h) * dv + i] = from_float<T>(pa_turned(get, i, dv, vcos ? style : PA_STYLE_NONE, vcos, vsin, tpos, -1.f));
}

// The same for heads whose keys are multiples of 8 elements and whose values are an even number: a block of W waves per (row, head), the
// waves taking the batches of 64 keys in turn and meeting in LDS in the order of the waves; a key's row is read 16 bytes at a time, a
// lane owns two neighbouring output elements (and the two 128 further on).
template <typename T, int W>
__global__ __launch_bounds__(W * TQK_WAVE)
void pooled_attention_rows_kernel(const T* __restrict__ q, const T* __restrict__ keys, const T* __restrict__ values, const int32_t* __restrict__ row_seq,
                                  const int32_t* __restrict__ row_pos, const int32_t* __restrict__ table, int width, int window, int pool, float scale,
                                  const float* __restrict__ sink, const float* __restrict__ vcos, const float* __restrict__ vsin, int style, int max_pos,
                                  T* __restrict__ out, int H, int G, int d, int dv, int page_rows) {
    __shared__ __attribute__((aligned(16))) float q_lds[PA_MAX_DIM];
    __shared__ float o_lds[W][PA_MAX_DIM];
    __shared__ float ml_lds[W][2];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const long long item = blockIdx.x;
    const long long r = item / H;
    const int h = (int)(item % H), g = h / (H / G);
    const int pos = row_pos[r];
    const int32_t* pages = table + (size_t)row_seq[r] * width;
    for (int i = threadIdx.x; i < d; i += W * TQK_WAVE) q_lds[i] = to_float(q[((size_t)r * H + h) * d + i]) * scale;
    __syncthreads();
    const int lo = max(0, pos - window + 1);
    const int n_blocks = pos - window + 1 >= pool ? (pos - window + 1) / pool : 0;
    const int n_all = n_blocks + (pos - lo + 1);
    float m = -INFINITY, l = 0.f;
    float acc[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
    for (int n0 = wave * TQK_WAVE; n0 < n_all; n0 += W * TQK_WAVE) {
        const int n = n0 + lane;
        long long row = -1;
        if (n < n_all) {
            int page, in_page;
            if (n < n_blocks) { page = pages[(n * pool + pool - 1) / TQK_PAGE]; in_page = pa_pooled_row(n, pool); }
            else { const int j = lo + (n - n_blocks); page = pages[j / TQK_PAGE]; in_page = j % TQK_PAGE; }
            row = ((long long)page * G + g) * page_rows + in_page;
        }
        float s = -INFINITY;
        if (row >= 0) {
            const T* kr = keys + (size_t)row * d;
            float d0 = 0.f, d1 = 0.f;
#pragma unroll 4
            for (int i = 0; i < d; i += 8) {
                const float4 qa = *reinterpret_cast<const float4*>(q_lds + i), qb = *reinterpret_cast<const float4*>(q_lds + i + 4);
                float k8[8];
                if (sizeof(T) == 2) {
                    const uint4 kv = *reinterpret_cast<const uint4*>(kr + i);
                    const uint32_t w4[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) { k8[2 * j] = __uint_as_float(w4[j] << 16); k8[2 * j + 1] = __uint_as_float(w4[j] & 0xffff0000u); }
                } else {
                    const float4 ka = *reinterpret_cast<const float4*>(kr + i), kb = *reinterpret_cast<const float4*>(kr + i + 4);
                    k8[0] = ka.x; k8[1] = ka.y; k8[2] = ka.z; k8[3] = ka.w; k8[4] = kb.x; k8[5] = kb.y; k8[6] = kb.z; k8[7] = kb.w;
                }
                d0 = fmaf(qa.x, k8[0], d0); d1 = fmaf(qa.y, k8[1], d1); d0 = fmaf(qa.z, k8[2], d0); d1 = fmaf(qa.w, k8[3], d1);
                d0 = fmaf(qb.x, k8[4], d0); d1 = fmaf(qb.y, k8[5], d1); d0 = fmaf(qb.z, k8[6], d0); d1 = fmaf(qb.w, k8[7], d1);
            }
            s = d0 + d1;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float corr = expf(m - m_new);
        const float p = row >= 0 ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(p);
        m = m_new;
        acc[0][0] *= corr; acc[0][1] *= corr; acc[1][0] *= corr; acc[1][1] *= corr;
        // eight keys at a time: their weights and rows from the lanes that hold them, then the eight loads together, then the sums
        const int n_here = min(TQK_WAVE, n_all - n0);
        for (int k = 0; k < n_here; k += 8) {
            float pk[8];
            const T* vr[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int kk = min(k + j, n_here - 1);
                const float pj = __shfl(p, kk, TQK_WAVE);
                pk[j] = k + j < n_here ? pj : 0.f;
                vr[j] = values + (size_t)__shfl(row, kk, TQK_WAVE) * dv;
            }
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const int i = c * 2 * TQK_WAVE + 2 * lane;
                if (i < dv) {
                    float v0[8], v1[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        if (sizeof(T) == 2) { const uint32_t vv = *reinterpret_cast<const uint32_t*>(vr[j] + i); v0[j] = __uint_as_float(vv << 16); v1[j] = __uint_as_float(vv & 0xffff0000u); }
                        else { const float2 vv = *reinterpret_cast<const float2*>(vr[j] + i); v0[j] = vv.x; v1[j] = vv.y; }
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        acc[c][0] = fmaf(pk[j], v0[j], acc[c][0]);
                        acc[c][1] = fmaf(pk[j], v1[j], acc[c][1]);
                    }
                }
            }
        }
    }
    // the waves meet: every one leaves its maximum, its sum and its part of the output; the first adds them up in their order
    if (lane == 0) { ml_lds[wave][0] = m; ml_lds[wave][1] = l; }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int i = c * 2 * TQK_WAVE + 2 * lane;
        if (i < dv) { o_lds[wave][i] = acc[c][0]; o_lds[wave][i + 1] = acc[c][1]; }
    }
    __syncthreads();
    if (wave != 0) return;
    float mt = sink ? sink[h] : -INFINITY;
    for (int w = 0; w < W; ++w) mt = fmaxf(mt, ml_lds[w][0]);
    float lt = sink ? expf(sink[h] - mt) : 0.f;
    float f[W];
    for (int w = 0; w < W; ++w) {
        f[w] = ml_lds[w][0] == -INFINITY ? 0.f : expf(ml_lds[w][0] - mt);
        lt = fmaf(ml_lds[w][1], f[w], lt);
    }
    const float inv = 1.f / lt;
    for (int i = lane; i < dv; i += TQK_WAVE) {
        float v = 0.f;
        for (int w = 0; w < W; ++w) v = fmaf(o_lds[w][i], f[w], v);
        q_lds[i] = v * inv;                 // (the query is no longer needed)
    }
    __builtin_amdgcn_wave_barrier();
    auto get = [&](int i) { return q_lds[i]; };
    const int tpos = min(pos, max_pos - 1);
    for (int i = lane; i < dv; i += TQK_WAVE)
        out[((size_t)r * H + h) * dv + i] = from_float<T>(pa_turned(get, i, dv, vcos ? style : PA_STYLE_NONE, vcos, vsin, tpos, -1.f));
}

extern "C" int tqk_pooled_attention_max_dim(void) { return PA_MAX_DIM; }
extern "C" int tqk_pooled_rows(int pool) { return pool > 0 ? (TQK_PAGE + pool - 1) / pool : 0; }

extern "C" int tqk_pooled_store(const void* qkv, int dtype, const float* q_weight, const float* k_weight, int normed, float eps, const float* cos,
                                const float* sin, int rot_dim, int style, const float* vcos, const float* vsin, int max_pos, const int32_t* tok_seq,
                                const int32_t* tok_pos, const int32_t* table, int width, void* keys, void* values, void* q_out, int n_tokens,
                                int heads, int kv_heads, int d, int dv, int pool, void* stream) {
    TQK_REQUIRE(qkv && tok_seq && tok_pos && table && keys && values && q_out, "tqk_pooled_store: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && d > 0 && dv > 0 && pool > 0 && width > 0, "tqk_pooled_store: bad sizes");
    TQK_REQUIRE(style == PA_STYLE_NONE || rot_dim == 0 || (cos && sin && rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= d && max_pos > 0), "tqk_pooled_store: bad rotation");
    TQK_REQUIRE(!vcos || (vsin && dv % 2 == 0 && style != PA_STYLE_NONE), "tqk_pooled_store: values are turned in the layout of the keys, over an even number of elements");
    if (n_tokens == 0) return 0;
    const long long items = (long long)n_tokens * (heads + 2 * kv_heads), blocks = (items + 3) / 4;
    TQK_REQUIRE(blocks <= 0x7fffffff, "tqk_pooled_store: too many rows");
    const int page_rows = TQK_PAGE + tqk_pooled_rows(pool);
    hipStream_t s = (hipStream_t)stream;
#define TQK_PS(T) pooled_store_kernel<T><<<(unsigned)blocks, 256, 0, s>>>((const T*)qkv, q_weight, k_weight, normed, eps, cos, sin, rot_dim, style, vcos, vsin, \
        max_pos, tok_seq, tok_pos, table, width, (T*)keys, (T*)values, (T*)q_out, items, heads, kv_heads, d, dv, page_rows)
    if (dtype == TQK_F32) TQK_PS(float);
    else if (dtype == TQK_BF16) TQK_PS(bf16_t);
    else return tqk_fail("tqk_pooled_store: unknown dtype %d", dtype);
#undef TQK_PS
    return tqk_check_launch("tqk_pooled_store");
}

extern "C" int tqk_pool_blocks(void* keys, void* values, int dtype, const int32_t* seq_start, const int32_t* seq_new, const int32_t* table, int width,
                               int n_seqs, int max_new, int pool, int kv_heads, int d, int dv, void* stream) {
    TQK_REQUIRE(keys && values && seq_start && seq_new && table, "tqk_pool_blocks: null pointer");
    TQK_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && kv_heads > 0 && kv_heads <= 65535 && max_new >= 0 && pool > 0 && d > 0 && dv > 0, "tqk_pool_blocks: bad sizes");
    if (n_seqs == 0) return 0;
    const int page_rows = TQK_PAGE + tqk_pooled_rows(pool);
    dim3 grid(max_new / pool + 1, kv_heads, n_seqs);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TQK_F32) pool_blocks_kernel<float><<<grid, 128, 0, s>>>((float*)keys, (float*)values, seq_start, seq_new, table, width, pool, kv_heads, d, dv, page_rows);
    else if (dtype == TQK_BF16) pool_blocks_kernel<bf16_t><<<grid, 128, 0, s>>>((bf16_t*)keys, (bf16_t*)values, seq_start, seq_new, table, width, pool, kv_heads, d, dv, page_rows);
    else return tqk_fail("tqk_pool_blocks: unknown dtype %d", dtype);
    return tqk_check_launch("tqk_pool_blocks");
}

extern "C" int tqk_pooled_attention(const void* q, const void* keys, const void* values, int dtype, const int32_t* row_seq, const int32_t* row_pos,
                                    const int32_t* table, int width, int window, int pool, float scale, const float* sink, const float* vcos,
                                    const float* vsin, int style, int max_pos, void* out, int n_rows, int heads, int kv_heads, int d, int dv,
                                    void* stream) {
    TQK_REQUIRE(q && keys && values && row_seq && row_pos && table && out, "tqk_pooled_attention: null pointer");
    TQK_REQUIRE(n_rows >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && window > 0 && pool > 0 && width > 0, "tqk_pooled_attention: bad sizes");
    TQK_REQUIRE(d > 0 && dv > 0 && d <= PA_MAX_DIM && dv <= PA_MAX_DIM, "tqk_pooled_attention: heads of %d and %d values, the kernel takes up to %d", d, dv, PA_MAX_DIM);
    TQK_REQUIRE(!vcos || (vsin && dv % 2 == 0 && max_pos > 0 && (style == PA_STYLE_HALVES || style == PA_STYLE_PAIRS)), "tqk_pooled_attention: bad rotation of the values");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * heads, blocks = (items + 3) / 4;
    TQK_REQUIRE(items <= 0x7fffffff, "tqk_pooled_attention: too many rows");
    const int page_rows = TQK_PAGE + tqk_pooled_rows(pool);
    hipStream_t s = (hipStream_t)stream;
    const int esize = dtype == TQK_BF16 ? 2 : 4;
    if (d % 8 == 0 && dv % 2 == 0 && (((uintptr_t)keys | (uintptr_t)values) & 15) == 0 && (dtype == TQK_BF16 || dtype == TQK_F32) && ((size_t)dv * esize) % 4 == 0) {
        // 32-bit steps keep one shape whatever the step holds (the order of the sums is then the position's alone); others deal a row's
        // keys out to more waves the fewer rows there are
#define TQK_PAR(T, W) pooled_attention_rows_kernel<T, W><<<(unsigned)items, W * TQK_WAVE, 0, s>>>((const T*)q, (const T*)keys, (const T*)values, row_seq, row_pos, table, \
        width, window, pool, scale, sink, vcos, vsin, style, max_pos, (T*)out, heads, kv_heads, d, dv, page_rows)
        if (dtype == TQK_F32) TQK_PAR(float, 4);
        else if (items >= 4096) TQK_PAR(bf16_t, 1);
        else if (items >= 1024) TQK_PAR(bf16_t, 4);
        else TQK_PAR(bf16_t, 8);
#undef TQK_PAR
        return tqk_check_launch("tqk_pooled_attention");
    }
#define TQK_PA(T) pooled_attention_kernel<T><<<(unsigned)blocks, 256, 0, s>>>((const T*)q, (const T*)keys, (const T*)values, row_seq, row_pos, table, width, window, \
        pool, scale, sink, vcos, vsin, style, max_pos, (T*)out, items, heads, kv_heads, d, dv, page_rows)
    if (dtype == TQK_F32) TQK_PA(float);
    else if (dtype == TQK_BF16) TQK_PA(bf16_t);
    else return tqk_fail("tqk_pooled_attention: unknown dtype %d", dtype);
#undef TQK_PA
    return tqk_check_launch("tqk_pooled_attention");
}
