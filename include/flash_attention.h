// Public C++ API and C-ABI of the MI355X (gfx950) causal flash attention:
// the forward, and a backward the reference does not have.  Keeps the name, argument order and meaning of the reference's
// include/flash_attention.h:12-24 with the HIP spellings of the platform
// types.  The caller owns all buffers; the call enqueues on `stream`, does not
// synchronise and allocates nothing.
#pragma once

#include <cstddef>

#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>

namespace dscuda {

// Fuses causal QK^T, online softmax and PV without materialising the T x T
// score matrix.  query/output BF16 [B,T,Hq,D], key/value BF16 [B,T,Hkv,D],
// natural-log logsumexp FP32 [B,Hq,T].  Hq must be divisible by Hkv (query
// head h reads kv head h / (Hq/Hkv)), T must be a positive multiple of 64
// (the reference's rule, kernels/attention/flash_attention/sm89_forward.cu:
// 226-232) and D must be 64 or 128 (the reference accepts 128 only).
void flash_attention_forward_cuda(
    __hip_bfloat16* output,
    float* logsumexp,
    const __hip_bfloat16* query,
    const __hip_bfloat16* key,
    const __hip_bfloat16* value,
    int batch_size,
    int sequence_length,
    int query_heads,
    int key_value_heads,
    int head_size,
    float scale,
    hipStream_t stream = nullptr);

// FP32 elements of workspace the backward needs (row statistics of every query head plus
// the BF16 dS blocks one pass hands to the other, for as many (batch, key/value head)
// pairs as one pass covers).  0 for shapes the backward rejects.
std::size_t flash_attention_backward_workspace_elements(
    int batch_size,
    int sequence_length,
    int query_heads,
    int key_value_heads,
    int head_size);

// Replaces, for the whole process, the 3 GiB that the dS blocks of one chunk of (batch,
// key/value head) pairs may take (0 restores it): set it before asking for the workspace
// size and leave it unchanged until the backward call has been issued.
void flash_attention_backward_set_workspace_limit(std::size_t bytes);

// Recompute-based backward of flash_attention_forward_cuda from the saved BF16 output and
// FP32 logsumexp; it has no counterpart in the reference (whose flash attention is forward
// only, include/flash_attention.h:12-24).  dQ [B,T,Hq,D], dK and dV [B,T,Hkv,D] are
// overwritten.  With grouped-query heads the gradient of a key/value head is the sum over
// the query heads that read it, accumulated by one workgroup in a fixed order: no atomics,
// bit-reproducible.  Any positive T (the forward's multiple-of-64 rule is not needed here).
void flash_attention_backward_cuda(
    __hip_bfloat16* query_gradient,
    __hip_bfloat16* key_gradient,
    __hip_bfloat16* value_gradient,
    const __hip_bfloat16* output_gradient,
    const __hip_bfloat16* output,
    const float* logsumexp,
    const __hip_bfloat16* query,
    const __hip_bfloat16* key,
    const __hip_bfloat16* value,
    float* workspace,
    int batch_size,
    int sequence_length,
    int query_heads,
    int key_value_heads,
    int head_size,
    float scale,
    hipStream_t stream = nullptr);

}  // namespace dscuda

// ---- C ABI (libdscuda_flash_attention_bench.so) -----------------------------
// Replaces reference benchmarks/bindings/flash_attention_bridge.cu:13-30.
extern "C" {

const char* dscuda_flash_last_error();  // flash_attention_bridge.cu:13-15

int dscuda_flash_forward(  // flash_attention_bridge.cu:17-30
    __hip_bfloat16* output, float* logsumexp,
    const __hip_bfloat16* query, const __hip_bfloat16* key, const __hip_bfloat16* value,
    int batch, int sequence, int query_heads, int key_value_heads, int dimension,
    float scale, hipStream_t stream);

// additive (no counterpart in the reference): see dscuda::flash_attention_backward_cuda above
std::size_t dscuda_flash_backward_workspace_elements(
    int batch, int sequence, int query_heads, int key_value_heads, int dimension);

void dscuda_flash_backward_set_workspace_limit(std::size_t bytes);

int dscuda_flash_backward(
    __hip_bfloat16* dquery, __hip_bfloat16* dkey, __hip_bfloat16* dvalue,
    const __hip_bfloat16* dout, const __hip_bfloat16* output, const float* logsumexp,
    const __hip_bfloat16* query, const __hip_bfloat16* key, const __hip_bfloat16* value,
    float* workspace,
    int batch, int sequence, int query_heads, int key_value_heads, int dimension,
    float scale, hipStream_t stream);

}  // extern "C"
