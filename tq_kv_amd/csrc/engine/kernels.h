// The entry points of the kernel library (csrc/tq_kernels.h) as the engine calls them: looked up
// by name at first use.  Launches raise with the library's message on failure; the queries
// (sizes of scratch memory, what a kernel takes) are plain host functions.
#pragma once
#include "core.h"

namespace tq {
namespace K {

#define TQ_KERNEL(name, ...) static Kernel<__VA_ARGS__> name("tqk_" #name)
#define TQ_QUERY(ret, name, ...) static KernelFn<ret(__VA_ARGS__)> name("tqk_" #name)
typedef const void* cptr;
typedef const int32_t* ci32;
typedef const float* cf32;

TQ_QUERY(int, abi_version);
TQ_QUERY(int, page_size);
TQ_QUERY(int, skinny_max_rows);
TQ_QUERY(int, mid_max_rows);
TQ_KERNEL(embed, cptr, int, ci32, int, int, int, float, float*, void*, cptr, float*, void*);
TQ_KERNEL(finish_logits, float*, int, int, cf32, float, float, void*);
TQ_KERNEL(random_normal, void*, int, long long, uint64_t, float, int, void*);
TQ_KERNEL(add_rmsnorm, float*, cptr, int, cptr, int, float, ci32, int, int, void*, int, void*);
TQ_KERNEL(add_rmsnorm_sums, float*, cf32, int, int, int, cptr, int, float, ci32, int, int, void*, int, void*);
TQ_QUERY(size_t, gemm_scratch_bytes, int, int, int, int, int, int, int);
TQ_KERNEL(gemm, cptr, int, cptr, int, cptr, int, void*, int, int, int, int, void*, void*);
TQ_KERNEL(fused_store, cptr, ci32, cf32, int, float, cptr, int, void*, int, int, int, int, void*);
TQ_KERNEL(fused_gated, cptr, cf32, int, float, cptr, int, void*, int, int, int, void*);
TQ_QUERY(int, fused_residual_parts, int, int);
TQ_KERNEL(fused_residual, cptr, cptr, int, float*, cptr, void*, float*, int, int, int, void*);
TQ_KERNEL(fused_residual_wf32, cptr, cptr, int, float*, cf32, void*, float*, int, int, int, void*);
TQ_KERNEL(fused_qkv, cptr, cf32, int, float, cptr, int, cptr, cf32, cf32, int, ci32, ci32, int, void*, void*, int, void*, int, int, int, int,
          int, void*);
TQ_QUERY(int, mid_splits, int, int, int);
TQ_KERNEL(mid_store, cptr, cptr, void*, int, int, int, int, void*, int, void*);
TQ_KERNEL(mid_gated, cptr, cptr, void*, int, int, int, void*, void*);
TQ_KERNEL(rope_store, cptr, int, cptr, int, cf32, cf32, int, int, int, ci32, ci32, ci32, int, int, void*, void*, int, void*, int, int, int, int,
          int, void*);
TQ_QUERY(int, rope_store_takes_sums, int, int, int, int, int, int);
TQ_KERNEL(rope_store_sums, cf32, int, cptr, int, cf32, cf32, int, int, int, ci32, ci32, ci32, int, int, void*, void*, int, void*, int, int, int,
          int, int, void*);
TQ_QUERY(int, attention_max_head_dim);
TQ_KERNEL(attention, cptr, cptr, cptr, int, ci32, ci32, ci32, int, int, int, int, float, void*, int, int, int, int, void*);
TQ_QUERY(int, attention_decode_supported, int);
TQ_KERNEL(attention_decode, cptr, cptr, cptr, ci32, ci32, int, int, int, int, float, int, void*, void*, void*, int, int, int, void*);
TQ_QUERY(int, attention_prefill_supported, int);
TQ_QUERY(int, attention_prefill_tile, int, int, int, int);
TQ_KERNEL(attention_prefill, cptr, cptr, cptr, ci32, ci32, int, int, int, ci32, ci32, ci32, int, int, ci32, ci32, int, float, void*, int, int,
          int, int, void*);
TQ_KERNEL(attention_prefill_capped, cptr, cptr, cptr, ci32, ci32, int, int, int, ci32, ci32, ci32, int, int, ci32, ci32, int, float, float, void*, int,
          int, int, int, void*);
TQ_KERNEL(swiglu, cptr, void*, int, int, int, void*);
TQ_KERNEL(gated_act, cptr, void*, int, int, int, int, float, float, void*);
TQ_KERNEL(fused_gated_act, cptr, cf32, int, float, cptr, int, void*, int, int, int, int, float, float, void*);
TQ_KERNEL(mid_gated_act, cptr, cptr, void*, int, int, int, void*, int, float, float, void*);
TQ_QUERY(int, latent_max_rank);
TQ_QUERY(int, latent_max_row);
TQ_KERNEL(latent_split, cptr, int, int, int, int, int, int, cptr, cptr, int, float, cf32, cf32, int, int, ci32, ci32, ci32, int, void*, void*, int,
          void*, float*, int, void*);
TQ_QUERY(int, latent_attention_mfma_supported, int, int);
TQ_QUERY(int, latent_attention_parts, int, int, int, int);
TQ_KERNEL(latent_attention_tiles, cf32, cptr, cptr, ci32, ci32, int, int, int, ci32, ci32, ci32, int, int, float, float*, int, int, int, int, void*);
TQ_KERNEL(latent_attention_mfma, cf32, cptr, cptr, ci32, ci32, ci32, int, int, int, int, float, float*, int, int, int, int, int, float*, float*, void*);
TQ_KERNEL(latent_absorb, cptr, int, cptr, int, int, int, int, int, cf32, cf32, int, int, ci32, float*, int, int, void*);
TQ_KERNEL(latent_attention, cf32, cptr, int, ci32, ci32, ci32, int, int, int, int, float, float*, int, int, int, int, void*);
TQ_KERNEL(latent_values, cf32, cptr, int, cf32, int, int, int, void*, int, int, void*);
TQ_QUERY(int, moe_max_experts);
TQ_QUERY(int, moe_max_tiles, int, int, int);
TQ_QUERY(int, moe_tile_rows);
TQ_QUERY(int, grouped_supported, int);
TQ_KERNEL(moe_product_mfma, cptr, ci32, cptr, long long, void*, int, int, int, int, float, float, ci32, ci32, ci32, ci32, int, int, void*);
TQ_KERNEL(head_product, cptr, int, long long, long long, cptr, void*, int, long long, long long, cf32, int, int, int, int, void*);
TQ_KERNEL(moe_route, cptr, int, cptr, int, int, int, int, float, int, int32_t*, float*, cptr, float*, int, void*);
TQ_KERNEL(moe_group, ci32, int, int, int, int, int32_t*, int32_t*, int32_t*, int32_t*, int32_t*, int32_t*, void*);
TQ_KERNEL(moe_product, cptr, int, ci32, cptr, int, long long, void*, int, int, int, int, float, float, ci32, ci32, ci32, ci32, int, void*);
TQ_KERNEL(moe_scale_rows, cptr, int, ci32, cf32, int, void*, float*, int, int, void*);
TQ_KERNEL(moe_combine, cptr, int, ci32, cf32, int, cptr, cf32, void*, int, int, void*);
TQ_KERNEL(pair_embed, cptr, int, int, long long, long long, ci32, ci32, ci32, ci32, ci32, int32_t*, float*, int, int, int, void*, int, void*);
TQ_KERNEL(remember_tokens, ci32, ci32, ci32, ci32, int32_t*, int, void*);
TQ_KERNEL(norm_add, float*, cptr, int, cptr, int, float, void*, int, int, void*);
TQ_KERNEL(unary_act, cptr, void*, int, long long, int, float, float, void*);
TQ_KERNEL(row_gate, cptr, int, cptr, int, float*, int, int, void*);
TQ_KERNEL(normed_rope_store, cptr, int, cptr, cptr, int, float, cf32, cf32, int, int, cptr, cptr, void*, ci32, ci32, ci32, int, void*, void*, void*,
          int, int, int, int, int, int, void*);
TQ_KERNEL(rope_norm_store, cptr, int, cptr, int, cf32, cf32, int, int, int, int, float, ci32, ci32, ci32, int, void*, void*, void*, int, int, int, int,
          int, int, void*);
TQ_QUERY(int, conv_max_taps);
TQ_QUERY(int, ssm_max_state);
TQ_KERNEL(conv_state, cptr, int, long long, cf32, cf32, cf32, int, int, cf32, long long, ci32, ci32, ci32, ci32, float*, int, int, void*);
TQ_KERNEL(conv_state_update, cptr, int, long long, cf32, int, float*, long long, ci32, ci32, ci32, int, int, void*);
TQ_KERNEL(rglru_gates, cf32, cf32, cf32, cf32, cf32, cf32, float*, float*, int, int, int, void*);
TQ_KERNEL(rglru_gates_any_order, cf32, cf32, cf32, cf32, cf32, cf32, float*, float*, int, int, int, void*);
TQ_KERNEL(conv_state_step, cptr, int, long long, cf32, cf32, cf32, int, int, float*, long long, ci32, ci32, float*, int, int, void*);
TQ_KERNEL(linear_scan, cf32, cf32, cptr, int, long long, cf32, float*, long long, ci32, ci32, ci32, void*, int, int, void*);
TQ_KERNEL(ssm_scan, cf32, long long, cptr, int, long long, cf32, cf32, cf32, float*, long long, ci32, ci32, ci32, float*, int, int, int, int, int, void*);
TQ_KERNEL(linear_chunks, cf32, cf32, cptr, int, long long, cf32, ci32, ci32, int, float*, float*, void*, int, int, void*);
TQ_KERNEL(chunk_carry, cf32, long long, int, float*, ci32, ci32, float*, long long, int, long long, void*);
TQ_KERNEL(ssm_steps, cptr, int, long long, cf32, cf32, float*, float*, int, int, void*);
TQ_KERNEL(ssm_chunks, cf32, long long, cf32, cf32, cf32, ci32, ci32, int, float*, float*, float*, int, int, int, int, int, void*);
TQ_KERNEL(gated_part_norm, cf32, cptr, int, long long, cf32, float, void*, int, int, int, void*);
TQ_KERNEL(add_rows, float*, cf32, long long, void*);
TQ_QUERY(int, attention_masked_max_dim);
TQ_QUERY(int, attention_masked_mfma_supported, int, int);
TQ_QUERY(int, attention_masked_mfma_tile, int, int, int, int, int);
TQ_KERNEL(attention_masked_mfma, cptr, cptr, cptr, ci32, ci32, int, int, int, int, float, float, cptr, int, ci32, ci32, ci32, int, int, int, int, void*, void*,
          void*, int, int, int, int, void*);
TQ_KERNEL(attention_masked, cptr, cptr, cptr, int, ci32, ci32, ci32, int, int, int, int, int, float, float, cptr, int, void*, int, int, int, int,
          int, void*);
TQ_QUERY(int, streams_max);
TQ_KERNEL(streams_fill, cf32, float*, int, int, int, void*);
TQ_KERNEL(streams_step, float*, int, cptr, int, cf32, cf32, cf32, cf32, cf32, float, float*, void*, int, int, int, int, void*);
TQ_KERNEL(add_layer_norm, float*, cptr, int, ci32, int, cf32, cf32, float, void*, int, int, int, void*);
TQ_KERNEL(token_shift, cf32, cf32, float*, long long, ci32, ci32, ci32, ci32, void*, int, int, int, int, void*);
TQ_KERNEL(shift_remember, cf32, float*, long long, ci32, ci32, ci32, int, int, void*);
TQ_QUERY(int, linear_attention_max_dim);
TQ_KERNEL(linear_attention, cptr, cptr, cptr, int, long long, cf32, long long, cf32, float, cf32, float, float, cf32, cf32, int, int, int, ci32, float*,
          long long, ci32, ci32, ci32, ci32, ci32, float*, float*, float*, int, int, int, int, int, void*);
TQ_KERNEL(head_norm_gate, cf32, cf32, float, cptr, int, long long, void*, int, int, int, int, void*);
TQ_QUERY(int, pooled_attention_max_dim);
TQ_QUERY(int, pooled_rows, int);
TQ_KERNEL(pooled_store, cptr, int, cf32, cf32, int, float, cf32, cf32, int, int, cf32, cf32, int, ci32, ci32, ci32, int, void*, void*, void*, int, int, int,
          int, int, int, void*);
TQ_KERNEL(pool_blocks, void*, void*, int, ci32, ci32, ci32, int, int, int, int, int, int, int, void*);
TQ_KERNEL(pooled_attention, cptr, cptr, cptr, int, ci32, ci32, ci32, int, int, int, float, cf32, cf32, cf32, int, int, void*, int, int, int, int, int,
          void*);
TQ_QUERY(int, pooled_attention_tiles_supported, int, int);
TQ_QUERY(int, pooled_attention_tile, int, int);
TQ_KERNEL(pooled_attention_tiles, cptr, cptr, cptr, ci32, ci32, int, int, int, float, cf32, cf32, cf32, int, int, ci32, ci32, ci32, int, int, void*, int, int,
          int, int, void*);
TQ_KERNEL(normed_pair_sum, cptr, cptr, int, cf32, cf32, float, float, void*, int, int, int, void*);
TQ_QUERY(int, argmax_scratch_floats, int, int);
TQ_KERNEL(argmax, cf32, int, int, int32_t*, float*, void*);
TQ_KERNEL(repeat_penalty, float*, int, int, ci32, ci32, ci32, int, ci32, int, float, void*);
TQ_KERNEL(append_history, ci32, ci32, int32_t*, int32_t*, int, int32_t*, int, void*);
TQ_QUERY(size_t, sample_scratch_bytes, int, int, int, float);
TQ_KERNEL(sample, cf32, int, int, float, int, float, cf32, int32_t*, void*, void*);
// rows of any kind gathered by index; a bias added to every row; a weight into the few-row kernels' order
TQ_KERNEL(gather_rows, cptr, ci32, int, long long, void*, void*);
TQ_KERNEL(add_bias, void*, int, cptr, int, int, int, void*);
TQ_KERNEL(pack_weight, cptr, void*, int, int, int, void*);
TQ_KERNEL(unpack_weight, cptr, void*, int, int, int, void*);
TQ_KERNEL(convert, cptr, int, void*, int, long long, void*);

#undef TQ_KERNEL
#undef TQ_QUERY

}  // namespace K
}  // namespace tq
