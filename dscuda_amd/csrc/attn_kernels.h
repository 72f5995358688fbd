// Internal launch interface between the public entry points (api_*.hip) and
// the kernel translation units.  Every function validates nothing: the entry
// points have already checked shapes.  All of them enqueue on `stream` and
// return without synchronising.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>

#include <cstddef>

namespace dscuda {

// attn_fwd.hip -- causal forward, per-head K/V (flash attention and MLA prefill).
// query [B,S,Hq,d_qk], key [B,S,Hkv,d_qk], value [B,S,Hkv,d_v], output
// [B,S,Hq,d_v], logsumexp [B,Hq,S].
void attention_forward_dispatch(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                                const __hip_bfloat16* key, const __hip_bfloat16* value, int batch_size,
                                int sequence_length, int query_heads, int key_value_heads, int qk_head_size,
                                int v_head_size, float scale, hipStream_t stream);

// attn_bwd.hip -- recompute backward of the above for Hq == Hkv.  The fp32
// workspace (attention_backward_workspace_elements floats) holds the per-row
// statistics and the bf16 dS blocks handed from the dK/dV kernel to the dQ pass.
std::size_t attention_backward_workspace_elements(int batch_size, int sequence_length, int heads, int kv_heads);

// Bytes the dS blocks of one chunk of (batch, key/value head) pairs may take (0: the built-in 3 GiB); process-wide.
void attention_backward_set_workspace_limit(std::size_t bytes);

void attention_backward_dispatch(__hip_bfloat16* query_gradient, __hip_bfloat16* key_gradient,
                                 __hip_bfloat16* value_gradient, const __hip_bfloat16* output_gradient,
                                 const __hip_bfloat16* output, const float* logsumexp, const __hip_bfloat16* query,
                                 const __hip_bfloat16* key, const __hip_bfloat16* value, float* workspace, int batch_size,
                                 int sequence_length, int heads, int kv_heads, int qk_head_size, int v_head_size,
                                 float scale, hipStream_t stream);

// rope.hip -- rotary position embedding, in place, on columns rope_offset .. rope_offset + rope_size - 1 of a
// [B, S, H, width] bf16 tensor (interleaved pairs; positions: per-sequence start positions or nullptr for 0).
void rope_apply_dispatch(__hip_bfloat16* tensor, const int* positions, int batch_size, int sequence_length, int heads,
                         int width, int rope_offset, int rope_size, float theta, hipStream_t stream);

// mla_projection.hip -- the per-head projections either side of absorbed attention: q_latent = q_nope W_UK and
// out = o_latent W_UV^T, both weights [heads, 128, 512] (head h at weight + h * weight_head_stride); token t, head h
// of a tensor at base + t * token_stride + h * head_stride (elements).
void mla_absorb_query_dispatch(__hip_bfloat16* query_latent, const __hip_bfloat16* query_nope,
                               const __hip_bfloat16* weight, long long tokens, int heads,
                               long long query_nope_token_stride, long long query_nope_head_stride,
                               long long query_latent_token_stride, long long query_latent_head_stride,
                               long long weight_head_stride, hipStream_t stream);
void mla_unabsorb_output_dispatch(__hip_bfloat16* output, const __hip_bfloat16* output_latent,
                                  const __hip_bfloat16* weight, long long tokens, int heads,
                                  long long output_latent_token_stride, long long output_latent_head_stride,
                                  long long output_token_stride, long long output_head_stride,
                                  long long weight_head_stride, hipStream_t stream);

// mla_absorbed.hip -- absorbed (C=512, R=64) causal forward and backward with
// one shared latent KV head.
void mla_absorbed_forward_dispatch(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query_latent,
                                   const __hip_bfloat16* query_rope, const __hip_bfloat16* kv_latent,
                                   const __hip_bfloat16* key_rope, int batch_size, int sequence_length, int heads,
                                   float scale, hipStream_t stream);

void mla_absorbed_backward_dispatch(__hip_bfloat16* query_latent_gradient, __hip_bfloat16* query_rope_gradient,
                                    __hip_bfloat16* kv_latent_gradient, __hip_bfloat16* key_rope_gradient,
                                    const __hip_bfloat16* output_gradient, const __hip_bfloat16* output,
                                    const float* logsumexp, const __hip_bfloat16* query_latent,
                                    const __hip_bfloat16* query_rope, const __hip_bfloat16* kv_latent,
                                    const __hip_bfloat16* key_rope, int batch_size, int sequence_length, int heads,
                                    float scale, hipStream_t stream);

// > 0: the key-gradient pass cuts its work by intervals of that many row tiles at any size; 0: its own choice.
void mla_absorbed_backward_set_key_interval_tiles(int tiles);

// mla_decode.hip -- absorbed single-token decode over a paged latent cache.  `plan` is
// the int table mla_decode_plan_dispatch writes for the same batch, heads and splits
// (mla_decode_plan_elements ints), or nullptr: the call then builds its own inside the
// workspace.
std::size_t mla_decode_plan_elements(int batch_size, int heads, int splits);

void mla_decode_plan_dispatch(int* plan, const int* cache_lengths, int batch_size, int heads, int splits,
                              hipStream_t stream);

void mla_decode_dispatch(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                         const __hip_bfloat16* paged_kv_cache, const int* block_table, const int* cache_lengths,
                         float* workspace, int* plan, int batch_size, int heads, int page_size,
                         int pages_per_sequence, int splits, float scale, hipStream_t stream);

}  // namespace dscuda
