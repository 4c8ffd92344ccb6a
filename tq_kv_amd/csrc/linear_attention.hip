// Linear attention with a decaying state: per head S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, with S of d rows (key
// channels) and dv columns in float32.  The decay a_t is one number per head (fixed) or one per key channel and token, formed here
// from a product z as sigmoid(z + bias)^(1/tau) = exp(logsigmoid(z + bias) / tau).  q and k may be turned by the position (tables of
// cos and sin, in halves or neighbouring pairs over the first rot_dim elements) and scaled on their way in; everything after the
// loads is float32.
//
// A block takes a head and a slab of columns; a thread a column and every RG-th row of it (rows i * RG + rg), so that a token's q, k
// and a are read from LDS at neighbouring addresses and a column's output is a sum over RG neighbouring lanes.  Tokens are staged in
// LDS eight at a time.  Three modes: scan (a sequence's tokens in order from the cache's state, which is written back), and for
// long steps chunks of consecutive tokens: local (every chunk from a zero state; its last state and the product of its decays are
// left for tqk_chunk_carry) and apply (every chunk again from the state it starts from, with the outputs).
//
// tqk_head_norm_gate: out = o / rms(o) (per head, times a weight over the head's columns if given) * silu(gate).
#include "common.h"
#include "tq_kernels.h"

#define LA_THREADS 256
#define LA_TB 8
enum { LA_SCAN = 0, LA_LOCAL = 1, LA_APPLY = 2 };
enum { LA_STYLE_HALVES = 1, LA_STYLE_PAIRS = 2 };

struct LaArgs {
    const void *q, *k, *v;
    long long stride;
    const float* z;
    long long z_stride;
    const float* z_bias;
    float inv_tau;
    const float* head_decay;
    float q_scale, k_scale;
    const float *cos, *sin;
    int rot_dim, style, max_pos;
    const int32_t* tok_pos;
    float* state;
    long long state_stride;
    const int32_t *cu, *seq_new, *seq_slot;
    const int32_t *chunk_row0, *chunk_count;
    float *chunk_state, *chunk_decay;
    float* out;
    int H, d, dv;
};

template <typename T, int RT, int MODE>
__global__ __launch_bounds__(LA_THREADS)
void linear_attention_kernel(LaArgs a, int rg_shift) {
    extern __shared__ float la_lds[];
    const int d = a.d, dv = a.dv, H = a.H;
    const int head = blockIdx.y, item = blockIdx.z;
    const int RG = 1 << rg_shift, CB = LA_THREADS >> rg_shift;
    const int rg = threadIdx.x & (RG - 1), col = blockIdx.x * CB + (threadIdx.x >> rg_shift);
    const bool col_ok = col < dv;
    int row0, count;
    if (MODE == LA_SCAN) { row0 = a.cu[item]; count = a.seq_new[item]; }
    else { row0 = a.chunk_row0[item]; count = a.chunk_count[item]; }
    if (count <= 0) return;
    const size_t per_head = (size_t)d * dv;
    float* sp = MODE == LA_SCAN ? a.state + (size_t)a.seq_slot[item] * a.state_stride + head * per_head
                                : a.chunk_state + ((size_t)item * H + head) * per_head;
    float S[RT], P[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        const int r = i * RG + rg;
        S[i] = (MODE != LA_LOCAL && r < d && col_ok) ? sp[(size_t)r * dv + col] : 0.f;
        P[i] = 1.f;
    }
    float* lq = la_lds;
    float* lk = la_lds + LA_TB * d;
    float* ld = la_lds + 2 * LA_TB * d;
    const T* qb = (const T*)a.q + (size_t)head * d;
    const T* kb = (const T*)a.k + (size_t)head * d;
    const T* vb = (const T*)a.v + (size_t)head * dv;
    const int half = a.rot_dim / 2;
    for (int t0 = 0; t0 < count; t0 += LA_TB) {
        const int nt = min(LA_TB, count - t0);
        __syncthreads();
        for (int e = threadIdx.x; e < nt * d; e += LA_THREADS) {
            const int tt = e / d, i = e - tt * d;
            const long long row = row0 + t0 + tt;
            const T* qr = qb + row * a.stride;
            const T* kr = kb + row * a.stride;
            float qv = to_float(qr[i]), kv = to_float(kr[i]);
            if (a.cos && i < a.rot_dim) {
                bool first;
                int pi, ai;
                if (a.style == LA_STYLE_HALVES) { first = i < half; pi = first ? i + half : i - half; ai = first ? i : i - half; }
                else { first = !(i & 1); pi = i ^ 1; ai = i >> 1; }
                const int pos = min(a.tok_pos[row], a.max_pos - 1);
                const float c = a.cos[(size_t)pos * half + ai], s = a.sin[(size_t)pos * half + ai];
                const float qp = to_float(qr[pi]), kp = to_float(kr[pi]);
                qv = first ? qv * c - qp * s : qv * c + qp * s;
                kv = first ? kv * c - kp * s : kv * c + kp * s;
            }
            lq[e] = qv * a.q_scale;
            lk[e] = kv * a.k_scale;
            float al;
            if (a.z) {
                const float zz = a.z[row * a.z_stride + (size_t)head * d + i] + a.z_bias[(size_t)head * d + i];
                const float ls = fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)));
                al = expf(ls * a.inv_tau);
            } else al = a.head_decay[head];
            ld[e] = al;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const long long row = row0 + t0 + tt;
            const float vv = col_ok ? to_float(vb[row * a.stride + col]) : 0.f;
            const float* q = lq + tt * d;
            const float* k = lk + tt * d;
            const float* al = ld + tt * d;
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const int r = i * RG + rg;
                if (r < d) {
                    S[i] = fmaf(al[r], S[i], k[r] * vv);
                    o = fmaf(S[i], q[r], o);
                    if (MODE == LA_LOCAL) P[i] *= al[r];
                }
            }
            if (MODE != LA_LOCAL) {
                for (int m = RG >> 1; m > 0; m >>= 1) o += __shfl_xor(o, m, TQK_WAVE);
                if (rg == 0 && col_ok) a.out[((size_t)row * H + head) * dv + col] = o;
            }
        }
    }
    if (MODE == LA_APPLY) return;
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        const int r = i * RG + rg;
        if (r < d && col_ok) sp[(size_t)r * dv + col] = S[i];
        if (MODE == LA_LOCAL && r < d && col == 0) a.chunk_decay[((size_t)item * H + head) * d + r] = P[i];
    }
}

// The same with a block of the state per thread: RT neighbouring rows by four neighbouring columns, for heads whose sizes are multiples of
// four.  A token costs a thread three 16-byte LDS reads per four rows (q, k and the decay) and one for its four values, for 4 RT state
// elements; rows beyond the head's (the padding up to RG * RT) stay zero.
template <typename T, int RT, int MODE>
__global__ __launch_bounds__(LA_THREADS)
void linear_attention_block_kernel(LaArgs a, int rg_shift, int cb) {
    extern __shared__ float la_lds[];
    const int d = a.d, dv = a.dv, H = a.H;
    const int head = blockIdx.y, item = blockIdx.z;
    const int RG = 1 << rg_shift, dpad = RG * RT;
    const int rg = threadIdx.x & (RG - 1), cg = threadIdx.x >> rg_shift;
    const int col0 = blockIdx.x * cb + cg * 4;
    const bool col_ok = cg * 4 < cb && col0 < dv;
    int row0, count;
    if (MODE == LA_SCAN) { row0 = a.cu[item]; count = a.seq_new[item]; }
    else { row0 = a.chunk_row0[item]; count = a.chunk_count[item]; }
    if (count <= 0) return;
    const size_t per_head = (size_t)d * dv;
    float* sp = MODE == LA_SCAN ? a.state + (size_t)a.seq_slot[item] * a.state_stride + head * per_head
                                : a.chunk_state + ((size_t)item * H + head) * per_head;
    float S[RT][4], P[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        const int r = rg * RT + i;
#pragma unroll
        for (int c = 0; c < 4; ++c) S[i][c] = (MODE != LA_LOCAL && r < d && col_ok) ? sp[(size_t)r * dv + col0 + c] : 0.f;
        P[i] = 1.f;
    }
    float* lq = la_lds;
    float* lk = lq + LA_TB * dpad;
    float* ld = lk + LA_TB * dpad;
    float* lv = ld + LA_TB * dpad;
    const T* qb = (const T*)a.q + (size_t)head * d;
    const T* kb = (const T*)a.k + (size_t)head * d;
    const T* vb = (const T*)a.v + (size_t)head * dv;
    const int half = a.rot_dim / 2;
    for (int t0 = 0; t0 < count; t0 += LA_TB) {
        const int nt = min(LA_TB, count - t0);
        __syncthreads();
        for (int e = threadIdx.x; e < nt * dpad; e += blockDim.x) {
            const int tt = e / dpad, i = e - tt * dpad;
            float qv = 0.f, kv = 0.f, al = 0.f;
            if (i < d) {
                const long long row = row0 + t0 + tt;
                const T* qr = qb + row * a.stride;
                const T* kr = kb + row * a.stride;
                qv = to_float(qr[i]);
                kv = to_float(kr[i]);
                if (a.cos && i < a.rot_dim) {
                    bool first;
                    int pi, ai;
                    if (a.style == LA_STYLE_HALVES) { first = i < half; pi = first ? i + half : i - half; ai = first ? i : i - half; }
                    else { first = !(i & 1); pi = i ^ 1; ai = i >> 1; }
                    const int pos = min(a.tok_pos[row], a.max_pos - 1);
                    const float c = a.cos[(size_t)pos * half + ai], s = a.sin[(size_t)pos * half + ai];
                    const float qp = to_float(qr[pi]), kp = to_float(kr[pi]);
                    qv = first ? qv * c - qp * s : qv * c + qp * s;
                    kv = first ? kv * c - kp * s : kv * c + kp * s;
                }
                qv *= a.q_scale;
                kv *= a.k_scale;
                if (a.z) {
                    const float zz = a.z[row * a.z_stride + (size_t)head * d + i] + a.z_bias[(size_t)head * d + i];
                    const float ls = fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)));
                    al = expf(ls * a.inv_tau);
                } else al = a.head_decay[head];
            }
            lq[e] = qv;
            lk[e] = kv;
            ld[e] = al;
        }
        for (int e = threadIdx.x; e < nt * cb; e += blockDim.x) {
            const int tt = e / cb, c = e - tt * cb, col = blockIdx.x * cb + c;
            lv[e] = col < dv ? to_float(vb[(row0 + t0 + tt) * a.stride + col]) : 0.f;
        }
        __syncthreads();
        if (cg * 4 < cb) {
            for (int tt = 0; tt < nt; ++tt) {
                const float4 vv = *reinterpret_cast<const float4*>(lv + tt * cb + cg * 4);
                const float v4[4] = {vv.x, vv.y, vv.z, vv.w};
                float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < RT; i += 4) {
                    const float4 q4 = *reinterpret_cast<const float4*>(lq + tt * dpad + rg * RT + i);
                    const float4 k4 = *reinterpret_cast<const float4*>(lk + tt * dpad + rg * RT + i);
                    const float4 a4 = *reinterpret_cast<const float4*>(ld + tt * dpad + rg * RT + i);
                    const float qq[4] = {q4.x, q4.y, q4.z, q4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, aa[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            S[i + j][c] = fmaf(aa[j], S[i + j][c], kk[j] * v4[c]);
                            o[c] = fmaf(S[i + j][c], qq[j], o[c]);
                        }
                        if (MODE == LA_LOCAL) P[i + j] *= aa[j];
                    }
                }
                if (MODE != LA_LOCAL) {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        for (int m = RG >> 1; m > 0; m >>= 1) o[c] += __shfl_xor(o[c], m, TQK_WAVE);
                    if (rg == 0 && col_ok) {
                        float* dst = a.out + ((size_t)(row0 + t0 + tt) * H + head) * dv + col0;
#pragma unroll
                        for (int c = 0; c < 4; ++c) dst[c] = o[c];
                    }
                }
            }
        }
    }
    if (MODE == LA_APPLY) return;
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        const int r = rg * RT + i;
        if (r < d && col_ok) {
#pragma unroll
            for (int c = 0; c < 4; ++c) sp[(size_t)r * dv + col0 + c] = S[i][c];
        }
        if (MODE == LA_LOCAL && r < d && col0 == 0 && col_ok) a.chunk_decay[((size_t)item * H + head) * d + r] = P[i];
    }
}

// out[t, h, j] = o[t, h, j] / sqrt(mean_j o[t, h]^2 + eps) * w[j] * silu(gate[t, h * dv + j]); a wave per (token, head)
template <typename TG, typename TO>
__global__ __launch_bounds__(256)
void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, float eps, const TG* __restrict__ gate, long long gate_stride,
                           TO* __restrict__ out, long long n_pairs, int H, int dv) {
    const long long pair = (long long)blockIdx.x * (256 / TQK_WAVE) + threadIdx.x / TQK_WAVE;
    if (pair >= n_pairs) return;
    const int lane = threadIdx.x % TQK_WAVE;
    const long long t = pair / H;
    const int h = (int)(pair % H);
    const float* orow = o + (size_t)pair * dv;
    float ss = 0.f;
    for (int j = lane; j < dv; j += TQK_WAVE) ss = fmaf(orow[j], orow[j], ss);
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)dv + eps);
    for (int j = lane; j < dv; j += TQK_WAVE) {
        const float g = gate ? to_float(gate[t * gate_stride + (size_t)h * dv + j]) : 0.f;
        float v = orow[j] * inv;
        if (w) v *= w[j];
        if (gate) v *= g / (1.f + expf(-g));
        out[(size_t)pair * dv + j] = from_float<TO>(v);
    }
}

extern "C" int tqk_linear_attention_max_dim(void) { return 512; }

extern "C" int tqk_linear_attention(const void* q, const void* k, const void* v, int act_dtype, long long stride, const float* z, long long z_stride,
                                    const float* z_bias, float inv_tau, const float* head_decay, float q_scale, float k_scale, const float* cos,
                                    const float* sin, int rot_dim, int style, int max_pos, const int32_t* tok_pos, float* state, long long state_stride,
                                    const int32_t* cu, const int32_t* seq_new, const int32_t* seq_slot, const int32_t* chunk_row0,
                                    const int32_t* chunk_count, float* chunk_state, float* chunk_decay, float* out, int mode, int n_items, int heads,
                                    int d, int dv, void* stream) {
    TQK_REQUIRE(q && k && v, "tqk_linear_attention: null pointer");
    TQK_REQUIRE((z && z_bias) || head_decay, "tqk_linear_attention: neither a decay per channel nor one per head");
    TQK_REQUIRE(mode >= LA_SCAN && mode <= LA_APPLY, "tqk_linear_attention: unknown mode %d", mode);
    TQK_REQUIRE(mode == LA_SCAN ? (state && cu && seq_new && seq_slot) : (chunk_row0 && chunk_count && chunk_state && chunk_decay),
                "tqk_linear_attention: mode %d lacks its arrays", mode);
    TQK_REQUIRE(mode == LA_LOCAL || out, "tqk_linear_attention: nothing to write to");
    TQK_REQUIRE(n_items >= 0 && n_items <= 65535 && heads > 0 && heads <= 65535 && d > 0 && dv > 0, "tqk_linear_attention: bad sizes");
    TQK_REQUIRE(d <= tqk_linear_attention_max_dim() && dv <= 65535, "tqk_linear_attention: heads of %d key channels, the kernel takes up to %d", d, tqk_linear_attention_max_dim());
    TQK_REQUIRE(!cos || (sin && tok_pos && rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= d && max_pos > 0 && (style == LA_STYLE_HALVES || style == LA_STYLE_PAIRS)),
                "tqk_linear_attention: bad rotation");
    if (n_items == 0) return 0;
    LaArgs a = {q, k, v, stride, z, z_stride, z_bias, inv_tau, head_decay, q_scale, k_scale, cos, sin, rot_dim, style, max_pos, tok_pos, state, state_stride,
                cu, seq_new, seq_slot, chunk_row0, chunk_count, chunk_state, chunk_decay, out, heads, d, dv};
    hipStream_t s = (hipStream_t)stream;
    if (d % 4 == 0 && dv % 4 == 0 && dv >= 16 && (((uintptr_t)out) & 15) == 0) {
        // a thread holds rt rows by four columns: rt = 16 where the head has the rows for it, and as many row groups as cover the head
        const int rt = d >= 64 ? 16 : d >= 32 ? 8 : 4;
        int shift = 0;
        while ((rt << shift) < d) ++shift;
        if ((1 << shift) <= TQK_WAVE) {
            const int groups = LA_THREADS >> shift;                        // column groups a block has threads for
            const int cb = 4 * (((dv + 3) / 4 < groups) ? (dv + 3) / 4 : groups);
            int threads = ((cb / 4) << shift);
            threads = (threads + TQK_WAVE - 1) / TQK_WAVE * TQK_WAVE;
            dim3 bgrid((dv + cb - 1) / cb, heads, n_items);
            const size_t blds = (size_t)LA_TB * (3 * (size_t)(rt << shift) + cb) * sizeof(float);
#define TQK_LAB(T, RT, MODE) linear_attention_block_kernel<T, RT, MODE><<<bgrid, threads, blds, s>>>(a, shift, cb)
#define TQK_LAB_MODE(T, RT) do { if (mode == LA_SCAN) TQK_LAB(T, RT, LA_SCAN); else if (mode == LA_LOCAL) TQK_LAB(T, RT, LA_LOCAL); else TQK_LAB(T, RT, LA_APPLY); } while (0)
#define TQK_LAB_ROWS(T) do { if (rt == 16) TQK_LAB_MODE(T, 16); else if (rt == 8) TQK_LAB_MODE(T, 8); else TQK_LAB_MODE(T, 4); } while (0)
            if (act_dtype == TQK_F32) TQK_LAB_ROWS(float);
            else if (act_dtype == TQK_BF16) TQK_LAB_ROWS(bf16_t);
            else return tqk_fail("tqk_linear_attention: unknown dtype %d", act_dtype);
#undef TQK_LAB_ROWS
#undef TQK_LAB_MODE
#undef TQK_LAB
            return tqk_check_launch("tqk_linear_attention");
        }
    }
    // the widest slab of columns (a power of two up to 128, no wider than the head needs) whose threads hold at most 64 rows each
    int cb = 16;
    while (cb < 128 && cb < dv) cb *= 2;
    while (cb > 4 && (d + LA_THREADS / cb - 1) / (LA_THREADS / cb) > 64) cb /= 2;
    const int rg = LA_THREADS / cb;
    int rg_shift = 0;
    while ((1 << rg_shift) < rg) ++rg_shift;
    const int rows = (d + rg - 1) / rg;
    TQK_REQUIRE(rows <= 64, "tqk_linear_attention: %d rows a thread", rows);
    dim3 grid((dv + cb - 1) / cb, heads, n_items);
    const size_t lds = (size_t)3 * LA_TB * d * sizeof(float);
#define TQK_LA(T, RT, MODE) linear_attention_kernel<T, RT, MODE><<<grid, LA_THREADS, lds, s>>>(a, rg_shift)
#define TQK_LA_MODE(T, RT) do { if (mode == LA_SCAN) TQK_LA(T, RT, LA_SCAN); else if (mode == LA_LOCAL) TQK_LA(T, RT, LA_LOCAL); else TQK_LA(T, RT, LA_APPLY); } while (0)
#define TQK_LA_ROWS(T) do { if (rows <= 1) TQK_LA_MODE(T, 1); else if (rows <= 2) TQK_LA_MODE(T, 2); else if (rows <= 4) TQK_LA_MODE(T, 4); \
        else if (rows <= 8) TQK_LA_MODE(T, 8); else if (rows <= 16) TQK_LA_MODE(T, 16); else if (rows <= 32) TQK_LA_MODE(T, 32); else TQK_LA_MODE(T, 64); } while (0)
    if (act_dtype == TQK_F32) TQK_LA_ROWS(float);
    else if (act_dtype == TQK_BF16) TQK_LA_ROWS(bf16_t);
    else return tqk_fail("tqk_linear_attention: unknown dtype %d", act_dtype);
#undef TQK_LA_ROWS
#undef TQK_LA_MODE
#undef TQK_LA
    return tqk_check_launch("tqk_linear_attention");
}

extern "C" int tqk_head_norm_gate(const float* o, const float* weight, float eps, const void* gate, int gate_dtype, long long gate_stride, void* out,
                                  int out_dtype, int n_tokens, int heads, int dv, void* stream) {
    TQK_REQUIRE(o && out, "tqk_head_norm_gate: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && heads > 0 && dv > 0, "tqk_head_norm_gate: bad sizes");
    const long long pairs = (long long)n_tokens * heads;
    if (pairs == 0) return 0;
    const long long blocks = (pairs + 3) / 4;
    TQK_REQUIRE(blocks <= 0x7fffffff, "tqk_head_norm_gate: too many rows");
    hipStream_t s = (hipStream_t)stream;
#define TQK_HNG(TG, TO) head_norm_gate_kernel<TG, TO><<<(unsigned)blocks, 256, 0, s>>>(o, weight, eps, (const TG*)gate, gate_stride, (TO*)out, pairs, heads, dv)
    if (gate_dtype == TQK_F32 && out_dtype == TQK_F32) TQK_HNG(float, float);
    else if (gate_dtype == TQK_BF16 && out_dtype == TQK_BF16) TQK_HNG(bf16_t, bf16_t);
    else if (gate_dtype == TQK_F32 && out_dtype == TQK_BF16) TQK_HNG(float, bf16_t);
    else if (gate_dtype == TQK_BF16 && out_dtype == TQK_F32) TQK_HNG(bf16_t, float);
    else return tqk_fail("tqk_head_norm_gate: unknown dtypes %d, %d", gate_dtype, out_dtype);
#undef TQK_HNG
    return tqk_check_launch("tqk_head_norm_gate");
}
