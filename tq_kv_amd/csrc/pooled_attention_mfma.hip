// The attention of pooled_attention.hip on the matrix cores, for steps that bring several tokens of a sequence (bfloat16 in, float32
// softmax): v_mfma_f32_16x16x32_bf16, scores^T[key][column] = K . Q^T and out^T[element][column] = V^T . P^T with P staying in the lanes'
// registers.
//
// A block of four waves takes a tile of consecutive queries of one sequence and one kv head; a wave takes 16 of the tile's queries for one
// of the query heads that share the kv head (as many heads side by side as the group has, up to four; the waves left over take the next
// 16 queries).  What the block's columns see together (the blocks in front of the last query's window, then the positions from the first
// query's window on) is walked 32 at a time: their keys staged in LDS as they lie, their values turned over ([element][key]) on the way,
// so that both products read 16-byte operands; the next 32 are asked for while these are worked on and wait in registers.  Every column
// has its own position and masks what it does not see.
//
// Key r of a 16-key score tile t is the chunk's key 8 (r / 4) + 4 t + r % 4: a lane's eight scores of the two tiles are then eight
// neighbouring keys, which is how the second product wants its operand.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

#define PM_WAVES 4
#define PM_CHUNK 64          // keys and blocks staged at a time; the products take them 32 at a time
#define PM_LOG2E 1.4426950408889634f
enum { PM_STYLE_HALVES = 1, PM_STYLE_PAIRS = 2 };

struct PooledTileArgs {
    const bf16_t *q, *keys, *values;
    const int32_t *tok_pos, *table;
    int width, window, pool;
    float scale;
    const float *sink, *vcos, *vsin;
    int style, max_pos;
    const int32_t *tile_seq, *tile_tok0, *tile_count;
    bf16_t* out;
    int H, G, d, dv, page_rows, heads_per_block, head_blocks;
};

__device__ __forceinline__ int pm_pooled_row(int b, int pool) {
    const int e = b * pool + pool - 1, page = e / TQK_PAGE;
    return TQK_PAGE + b - (page * TQK_PAGE) / pool;
}

template <int KB, int DB>
__global__ __launch_bounds__(PM_WAVES * TQK_WAVE)
void pooled_attention_tiles_kernel(const PooledTileArgs a) {
    constexpr int D = KB * 32, DV = DB * 16, KROW = D + 8, VROW = PM_CHUNK + 8;
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[PM_CHUNK * KROW];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[DV * VROW];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int tile = blockIdx.x, g = blockIdx.y / a.head_blocks, hb = blockIdx.y % a.head_blocks;
    const int hpb = a.heads_per_block, group = a.H / a.G;
    const int seq = a.tile_seq[tile], tok0 = a.tile_tok0[tile], count = a.tile_count[tile];
    // the sequence's pages, once, where every later lookup is a read of LDS (a key's load then waits for one answer of memory, not two)
    extern __shared__ int32_t pages[];
    const int32_t* table_row = a.table + (size_t)seq * a.width;
    const int pos0 = a.tok_pos[tok0], pos_last = pos0 + count - 1;
    for (int i = threadIdx.x; i <= pos_last / TQK_PAGE && i < a.width; i += PM_WAVES * TQK_WAVE) pages[i] = table_row[i];
    __syncthreads();
    // what the block's columns see together
    const int lo_min = max(0, pos0 - a.window + 1);
    const int nb_max = pos_last - a.window + 1 >= a.pool ? (pos_last - a.window + 1) / a.pool : 0;
    const int n_all = nb_max + (pos_last - lo_min + 1);
    // this wave's columns
    const int hq = hb * hpb + wave % hpb, qt = wave / hpb;
    const bool wave_on = hq < group && qt * 16 < count;
    const int h = g * group + hq;
    const int col = lane & 15, lg = lane >> 4;
    const int my = qt * 16 + col;                      // the column's query among the tile's
    const bool col_on = wave_on && my < count;
    const int pos = pos0 + my;
    const int lo = max(0, pos - a.window + 1);
    const int nb = pos - a.window + 1 >= a.pool ? (pos - a.window + 1) / a.pool : 0;
    bf16x8_t bq[KB];
    {
        const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
        const bf16_t* qr = a.q + ((size_t)(tok0 + (col_on ? my : 0)) * a.H + (wave_on ? h : 0)) * D;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(qr + kb * 32 + lg * 8);
            bq[kb] = col_on ? v : zero;
        }
    }
    const float scale = a.scale * PM_LOG2E;
    float m = -INFINITY, l = 0.f;
    floatx4_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o[db] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    // The row (among all rows of the pages) of item n of what the block sees, or -1 beyond its end.
    auto row_at = [&](int n) -> long long {
        if (n >= n_all) return -1;
        int page, in_page;
        if (n < nb_max) { page = pages[(n * a.pool + a.pool - 1) / TQK_PAGE]; in_page = pm_pooled_row(n, a.pool); }
        else { const int j = lo_min + (n - nb_max); page = pages[j / TQK_PAGE]; in_page = j % TQK_PAGE; }
        return ((long long)page * a.G + g) * a.page_rows + in_page;
    };
    // A thread's pieces of a chunk: 16 bytes of a key row and of a value row each, KP and VP of them; asked for one chunk ahead and
    // held in registers while the chunk before is worked on.
    constexpr int NT = PM_WAVES * TQK_WAVE, KP = (PM_CHUNK * (D / 8) + NT - 1) / NT, VP = (PM_CHUNK * (DV / 8) + NT - 1) / NT;
    uint4 kreg[KP], vreg[VP];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int e = threadIdx.x + i * NT, r = e / (D / 8), c = e % (D / 8);
            kreg[i] = uint4{0u, 0u, 0u, 0u};
            if (e < PM_CHUNK * (D / 8)) {
                const long long row = row_at(n0 + r);
                if (row >= 0) kreg[i] = *reinterpret_cast<const uint4*>(a.keys + (size_t)row * D + c * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int e = threadIdx.x + i * NT, r = e % PM_CHUNK, c = e / PM_CHUNK;
            vreg[i] = uint4{0u, 0u, 0u, 0u};
            if (e < PM_CHUNK * (DV / 8)) {
                const long long row = row_at(n0 + r);
                if (row >= 0) vreg[i] = *reinterpret_cast<const uint4*>(a.values + (size_t)row * DV + c * 8);
            }
        }
    };
    fetch(0);
    for (int n0 = 0; n0 < n_all; n0 += PM_CHUNK) {
        __syncthreads();
        // keys as they lie; values turned over: [element][key]
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int e = threadIdx.x + i * NT, r = e / (D / 8), c = e % (D / 8);
            if (e < PM_CHUNK * (D / 8)) *reinterpret_cast<uint4*>(k_lds + r * KROW + c * 8) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int e = threadIdx.x + i * NT, r = e % PM_CHUNK, c = e / PM_CHUNK;
            if (e < PM_CHUNK * (DV / 8)) {
                const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v_lds[(c * 8 + 2 * j) * VROW + r].bits = (uint16_t)(w[j] & 0xffffu);
                    v_lds[(c * 8 + 2 * j + 1) * VROW + r].bits = (uint16_t)(w[j] >> 16);
                }
            }
        }
        __syncthreads();
        if (n0 + PM_CHUNK < n_all) fetch(n0 + PM_CHUNK);
        if (!wave_on) continue;
        for (int hh = 0; hh < PM_CHUNK / 32 && n0 + 32 * hh < n_all; ++hh) {
            // scores^T of the chunk's 32 keys against the wave's 16 columns
            floatx4_t s[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
                const int key = 32 * hh + 8 * (col >> 2) + 4 * t + (col & 3);           // the key this lane's row of the operand holds
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(k_lds + key * KROW + kb * 32 + lg * 8);
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, bq[kb], s[t], 0, 0, 0);
                }
            }
            // the lane's eight scores are keys 8 lg .. 8 lg + 7 of the chunk, for column col
            float sc[8];
            float top = -INFINITY;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int n = n0 + 32 * hh + 8 * lg + j;
                bool seen = col_on && n < n_all;
                if (n < nb_max) seen = seen && n < nb;
                else { const int jj = lo_min + (n - nb_max); seen = seen && jj >= lo && jj <= pos; }
                sc[j] = seen ? s[j >> 2][j & 3] * scale : -INFINITY;
                top = fmaxf(top, sc[j]);
            }
            top = fmaxf(top, __shfl_xor(top, 16, TQK_WAVE));
            top = fmaxf(top, __shfl_xor(top, 32, TQK_WAVE));
            const float m_new = fmaxf(m, top);
            const float base = m_new == -INFINITY ? 0.f : m_new;
            const float corr = __builtin_amdgcn_exp2f(m - base);             // m = -inf: 0
            float sum = 0.f;
            bf16x8_t pb;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const __bf16 p = (__bf16)__builtin_amdgcn_exp2f(sc[j] - base);
                pb[j] = p;
                sum += (float)p;
            }
            sum += __shfl_xor(sum, 16, TQK_WAVE);
            sum += __shfl_xor(sum, 32, TQK_WAVE);
            l = l * corr + sum;
            m = m_new;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                o[db] *= corr;
                const bf16x8_t av = *reinterpret_cast<const bf16x8_t*>(v_lds + (db * 16 + col) * VROW + 32 * hh + lg * 8);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb, o[db], 0, 0, 0);
            }
        }
    }
    if (!col_on) return;
    if (a.sink) {
        const float sv = a.sink[h] * PM_LOG2E, m_new = fmaxf(m, sv);
        const float corr = __builtin_amdgcn_exp2f(m - m_new);
        l = l * corr + __builtin_amdgcn_exp2f(sv - m_new);
#pragma unroll
        for (int db = 0; db < DB; ++db) o[db] *= corr;
    }
    const float inv = 1.f / l;
    // the lane holds elements 16 db + 4 lg + i of column col: turned back by the column's position, then stored
    bf16_t* dst = a.out + ((size_t)(tok0 + my) * a.H + h) * DV;
    const int tpos = min(pos, a.max_pos - 1);
    const int half = DV / 2;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = o[db][i] * inv;
        if (a.vcos) {
            if (a.style == PM_STYLE_PAIRS) {
#pragma unroll
                for (int i = 0; i < 4; i += 2) {
                    const int ai = (db * 16 + lg * 4 + i) >> 1;
                    const float c = a.vcos[(size_t)tpos * half + ai], sn = a.vsin[(size_t)tpos * half + ai];
                    const float x = v[i], y = v[i + 1];
                    v[i] = x * c + y * sn;
                    v[i + 1] = y * c - x * sn;
                }
            } else if (db < DB / 2) {
                // the partner of element e is e + DV / 2: the same lane, DB / 2 further on
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int ai = db * 16 + lg * 4 + i;
                    const float c = a.vcos[(size_t)tpos * half + ai], sn = a.vsin[(size_t)tpos * half + ai];
                    const float x = v[i], y = o[db + DB / 2][i] * inv;
                    v[i] = x * c + y * sn;
                    o[db + DB / 2][i] = (y * c - x * sn) / inv;
                }
            }
        }
        uint2 packed;
        packed.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
        packed.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
        *reinterpret_cast<uint2*>(dst + db * 16 + lg * 4) = packed;
    }
}

extern "C" int tqk_pooled_attention_tiles_supported(int d, int dv) {
    // (what a block stages of keys and values at a time stays below 60 KB of LDS)
    return d % 32 == 0 && d <= 256 && dv % 32 == 0 && dv <= 256 && 2 * (PM_CHUNK * (d + 8) + dv * (PM_CHUNK + 8)) <= 60 * 1024 ? 1 : 0;
}

// queries a tile of the step should hold: 16 for every wave that is left once the heads of a group have theirs
extern "C" int tqk_pooled_attention_tile(int heads, int kv_heads) {
    const int group = heads / (kv_heads > 0 ? kv_heads : 1);
    const int hpb = group >= 4 ? 4 : group >= 2 ? 2 : 1;
    return 16 * (PM_WAVES / hpb);
}

extern "C" int tqk_pooled_attention_tiles(const void* q, const void* keys, const void* values, const int32_t* tok_pos, const int32_t* table, int width,
                                          int window, int pool, float scale, const float* sink, const float* vcos, const float* vsin, int style,
                                          int max_pos, const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count, int n_tiles,
                                          int tile_queries, void* out, int heads, int kv_heads, int d, int dv, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && table && tile_seq && tile_tok0 && tile_count && out, "tqk_pooled_attention_tiles: null pointer");
    TQK_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && window > 0 && pool > 0 && width > 0, "tqk_pooled_attention_tiles: bad sizes");
    TQK_REQUIRE(tqk_pooled_attention_tiles_supported(d, dv), "tqk_pooled_attention_tiles: head sizes %d and %d are not taken", d, dv);
    TQK_REQUIRE(tile_queries == tqk_pooled_attention_tile(heads, kv_heads), "tqk_pooled_attention_tiles: tiles of %d queries, the kernel takes %d for these heads",
                tile_queries, tqk_pooled_attention_tile(heads, kv_heads));
    TQK_REQUIRE(!vcos || (vsin && max_pos > 0 && (style == PM_STYLE_HALVES || style == PM_STYLE_PAIRS)), "tqk_pooled_attention_tiles: bad rotation of the values");
    if (n_tiles <= 0) return 0;
    const int group = heads / kv_heads;
    const int hpb = group >= 4 ? 4 : group >= 2 ? 2 : 1;
    const int head_blocks = (group + hpb - 1) / hpb;
    TQK_REQUIRE((long long)kv_heads * head_blocks <= 65535, "tqk_pooled_attention_tiles: too many heads");
    PooledTileArgs a = {(const bf16_t*)q, (const bf16_t*)keys, (const bf16_t*)values, tok_pos, table, width, window, pool, scale, sink, vcos, vsin, style, max_pos,
                        tile_seq, tile_tok0, tile_count, (bf16_t*)out, heads, kv_heads, d, dv, TQK_PAGE + tqk_pooled_rows(pool), hpb, head_blocks};
    dim3 grid(n_tiles, kv_heads * head_blocks);
    hipStream_t s = (hipStream_t)stream;
    TQK_REQUIRE(width <= 8192, "tqk_pooled_attention_tiles: a page table of %d entries a sequence, the kernel takes 8192", width);
    const size_t lds = (size_t)width * sizeof(int32_t);
#define TQK_PT(KB, DB) pooled_attention_tiles_kernel<KB, DB><<<grid, PM_WAVES * TQK_WAVE, lds, s>>>(a)
#define TQK_PT_DB(KB) do { switch (dv / 32) { case 1: TQK_PT(KB, 2); break; case 2: TQK_PT(KB, 4); break; case 3: TQK_PT(KB, 6); break; case 4: TQK_PT(KB, 8); break; \
        case 5: TQK_PT(KB, 10); break; case 6: TQK_PT(KB, 12); break; case 7: TQK_PT(KB, 14); break; default: TQK_PT(KB, 16); break; } } while (0)
    switch (d / 32) {
        case 1: TQK_PT_DB(1); break;
        case 2: TQK_PT_DB(2); break;
        case 3: TQK_PT_DB(3); break;
        case 4: TQK_PT_DB(4); break;
        case 5: TQK_PT_DB(5); break;
        case 6: TQK_PT_DB(6); break;
        case 7: TQK_PT_DB(7); break;
        default: TQK_PT_DB(8); break;
    }
#undef TQK_PT_DB
#undef TQK_PT
    return tqk_check_launch("tqk_pooled_attention_tiles");
}
