// Public C++ API and C-ABI of the MI355X (gfx950) Multi-head Latent Attention
// kernels.  The first four functions keep the names, argument order and
// meaning of the reference's include/mla.h:18-81 with the HIP spellings of
// the two platform types (hipStream_t, __hip_bfloat16: both binary-identical
// to the reference's for a ctypes / dlsym caller).  The *_prefill_* functions
// are additive: the per-head (128 nope + 64 rope | 128 value) form has no
// counterpart in the reference.
//
// Conventions shared by every entry point:
//   * all activation / gradient buffers are BF16, statistics (logsumexp,
//     workspaces) are FP32, natural-log logsumexp of the *scaled* scores;
//   * the caller owns every buffer, including workspaces; the library
//     allocates nothing and keeps no state between calls;
//   * work is enqueued on `stream` without synchronising, so calls may be
//     captured into a HIP graph;
//   * invalid arguments throw std::invalid_argument / std::runtime_error
//     before anything is launched; the C-ABI wrappers turn that into status 1
//     plus a thread-local message.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>

#include <cstddef>

namespace dscuda {

constexpr int MLA_KV_RANK = 512;   // reference include/mla.h:10
constexpr int MLA_ROPE_SIZE = 64;  // reference include/mla.h:11

// Absorbed-query causal MLA forward.  Replaces reference include/mla.h:18-31.
// query_latent [B,T,H,C], query_rope [B,T,H,R], kv_latent [B,T,C], key_rope
// [B,T,R], output [B,T,H,C], logsumexp [B,H,T].  C must be 512 and R 64; B, T
// and H are free, T need not be a multiple of any tile.
void mla_compressed_attention_forward_cuda(
    __hip_bfloat16* output,
    float* logsumexp,
    const __hip_bfloat16* query_latent,
    const __hip_bfloat16* query_rope,
    const __hip_bfloat16* kv_latent,
    const __hip_bfloat16* key_rope,
    int batch_size,
    int sequence_length,
    int heads,
    int kv_rank,
    int rope_size,
    float scale,
    hipStream_t stream = nullptr);

// Absorbed-query MLA backward, recomputing probabilities from the saved FP32
// logsumexp.  Replaces reference include/mla.h:35-53.  The four gradient
// buffers are overwritten, the caller passes no workspace, and the result does
// not depend on timing: every gradient element is written by one thread and
// every sum has a fixed order (the reference's ownership rule,
// kernels/attention/mla/sm89.cu:2, kept as determinism).  Until the last of the
// call's launches the two query-gradient buffers hold intermediate values (row
// statistics, partial key gradients); both must be aligned to 16 bytes.
void mla_compressed_attention_backward_cuda(
    __hip_bfloat16* query_latent_gradient,
    __hip_bfloat16* query_rope_gradient,
    __hip_bfloat16* kv_latent_gradient,
    __hip_bfloat16* key_rope_gradient,
    const __hip_bfloat16* output_gradient,
    const __hip_bfloat16* output,
    const float* logsumexp,
    const __hip_bfloat16* query_latent,
    const __hip_bfloat16* query_rope,
    const __hip_bfloat16* kv_latent,
    const __hip_bfloat16* key_rope,
    int batch_size,
    int sequence_length,
    int heads,
    int kv_rank,
    int rope_size,
    float scale,
    hipStream_t stream = nullptr);

// FP32 elements of decode workspace.  Replaces reference include/mla.h:57-61;
// same formula, B*H*splits*(C+2), so buffers sized by either library fit.
std::size_t mla_decode_workspace_elements(
    int batch_size,
    int heads,
    int splits,
    int kv_rank);

// Absorbed decode of one packed BF16 query [B,1,H,C+R] against a paged cache
// [blocks,page,1,C+R] with block table [B,pages_per_sequence] and per-sequence
// lengths (>= 1).  Replaces reference include/mla.h:63-81.  `splits` bounds
// how finely a sequence may be partitioned (and with it the workspace); the
// result does not depend on it.  The workspace (mla_decode_workspace_elements
// floats, 16-byte aligned) needs no initialisation.  Any batch size.
void mla_decode_forward_cuda(
    __hip_bfloat16* output,
    float* logsumexp,
    const __hip_bfloat16* query,
    const __hip_bfloat16* paged_kv_cache,
    const int* block_table,
    const int* cache_lengths,
    float* workspace,
    int batch_size,
    int heads,
    int kv_rank,
    int rope_size,
    int page_size,
    int pages_per_sequence,
    int splits,
    float scale,
    hipStream_t stream = nullptr);

// ---- additive: a tuning knob of mla_compressed_attention_backward_cuda (no counterpart in
// the reference) -----------------------------------------------------------------------
//
// The key-gradient pass cuts its (key block, row tile) visits in one of two ways: into
// equal ranges, or -- when the query and dO rows of a batch element outgrow the caches --
// into (interval of row tiles, key block) items so that the workgroups running at one time
// walk the same rows.  tiles > 0 forces the second cut with that many 32-row tiles per
// interval at any size (as far as the partial-result slots inside dq_latent allow); 0, the
// default, leaves the choice to the library.  Process-wide; the results do not depend on it
// beyond the order of fp32 summation.
void mla_backward_set_key_interval_tiles(int tiles);

// ---- additive: a decode plan that outlives one call (no counterpart in the reference's
// kernels; the pattern of FlashMLA's get_mla_metadata, reference/python/flashmla.py:41-63) --
//
// Every decode call first turns the cache lengths into a small table: the tile
// prefix of the batch and its cut into one range per workgroup.
// mla_decode_forward_cuda derives that table from the lengths on every call (for
// the merge it leaves a copy inside its workspace).  A caller that decodes several
// layers (or steps) over the same lengths builds it once:
//     plan = device buffer of mla_decode_plan_elements(B, H, splits, C) ints
//     mla_decode_plan_cuda(plan, lengths, B, H, C, splits, stream)
//     for each layer: mla_decode_forward_planned_cuda(..., workspace, plan, ...)
// The plan depends on the lengths, B, H and splits (all must be the same in the
// calls that use it) and on the compute-unit count of the device that built it, and
// on nothing else.  mla_decode_plan_elements is plain arithmetic on its arguments
// (no device is asked, so it can be called on a host without a GPU): room for the
// plan of any device, 0 for arguments that admit no plan.
// The calls only read it: any number of them may share one plan, in any order and
// on any streams (each with a workspace of its own).
std::size_t mla_decode_plan_elements(
    int batch_size,
    int heads,
    int splits,
    int kv_rank);

void mla_decode_plan_cuda(
    int* plan,
    const int* cache_lengths,
    int batch_size,
    int heads,
    int kv_rank,
    int splits,
    hipStream_t stream = nullptr);

void mla_decode_forward_planned_cuda(
    __hip_bfloat16* output,
    float* logsumexp,
    const __hip_bfloat16* query,
    const __hip_bfloat16* paged_kv_cache,
    const int* block_table,
    const int* cache_lengths,
    float* workspace,
    int* plan,
    int batch_size,
    int heads,
    int kv_rank,
    int rope_size,
    int page_size,
    int pages_per_sequence,
    int splits,
    float scale,
    hipStream_t stream = nullptr);

// Bytes of the workspace built into the library for mla_decode_forward_static
// (one copy per GPU the library is loaded on, held until the process ends).
constexpr std::size_t MLA_DECODE_STATIC_SCRATCH_BYTES = std::size_t(64) << 20;

// mla_decode_forward_cuda for callers that cannot allocate or pass a workspace
// (code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc).  No counterpart in the reference.  Same arguments without the
// workspace: the partial results and the plan live in a fixed array inside the
// library, and the call performs no allocation of any kind.  Sizes for which
// batch*heads*splits*(kv_rank+2) floats exceed MLA_DECODE_STATIC_SCRATCH_BYTES
// are rejected with std::invalid_argument (lower `splits`: the result does not
// depend on it).  All calls on one GPU share that GPU's array: calls that
// overlap in time on one GPU (different streams or threads) race; calls in
// stream order do not, and nothing has to be cleared between them.  The first
// call on a device looks up the array's address and must not be made under
// stream capture.
void mla_decode_forward_static(
    __hip_bfloat16* output,
    float* logsumexp,
    const __hip_bfloat16* query,
    const __hip_bfloat16* paged_kv_cache,
    const int* block_table,
    const int* cache_lengths,
    int batch_size,
    int heads,
    int kv_rank,
    int rope_size,
    int page_size,
    int pages_per_sequence,
    int splits,
    float scale,
    hipStream_t stream = nullptr);

// ---- additive: per-head MLA prefill (no counterpart in the reference) ------
//
// query/key [B,S,H,d_qk] with the rope slice stored after the nope slice,
// value/output [B,S,H,d_v], logsumexp [B,H,S]; causal.  Supported head
// geometries: (d_qk,d_v) = (192,128), (128,128), (64,64).
void mla_prefill_forward_cuda(
    __hip_bfloat16* output,
    float* logsumexp,
    const __hip_bfloat16* query,
    const __hip_bfloat16* key,
    const __hip_bfloat16* value,
    int batch_size,
    int sequence_length,
    int heads,
    int qk_head_size,
    int v_head_size,
    float scale,
    hipStream_t stream = nullptr);

// FP32 elements of workspace the prefill backward needs: per-row statistics
// (logsumexp in log2 units and delta = sum(dO * O), 128 floats per 64-query
// tile) followed by the BF16 dS blocks the key/value-gradient pass hands to the
// query-gradient pass, 16 KB per causal (128-key block, 64-query tile) pair --
// about S*S bytes per (batch, head), for as many (batch, head) pairs at a time as
// fit 3 GiB (at least one): the two passes run over the pairs in chunks that share
// that set of blocks.  0 for non-positive sizes.
std::size_t mla_prefill_backward_workspace_elements(
    int batch_size,
    int sequence_length,
    int heads,
    int qk_head_size,
    int v_head_size);

// Replaces, for the whole process, the 3 GiB that the dS blocks of one chunk of
// (batch, head) pairs may take (0 restores it): a caller short of memory trades
// more launches for a smaller workspace.  Set it before asking for the workspace
// size and leave it unchanged until the backward call that uses that workspace has
// been issued.  No counterpart in the reference.
void mla_prefill_backward_set_workspace_limit(std::size_t bytes);

// Recompute-based backward of mla_prefill_forward_cuda from the saved BF16
// output and FP32 logsumexp.  dQ/dK [B,S,H,d_qk] and dV [B,S,H,d_v] are
// overwritten; every gradient row has exactly one writer (no atomics), dQ is
// produced by its own pass over the key blocks.
void mla_prefill_backward_cuda(
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
    int heads,
    int qk_head_size,
    int v_head_size,
    float scale,
    hipStream_t stream = nullptr);

// Rotary position embedding in place on columns rope_offset .. rope_offset + rope_size - 1 of
// every row of a [batch, sequence, heads, width] BF16 tensor: within the slice, columns
// (2i, 2i + 1) are rotated by position * theta^(-2i / rope_size), position = s +
// positions[b] (positions == nullptr: s).  The step before the attention kernels of an MLA
// layer -- q_rope [B,S,H,64] and k_rope [B,S,1,64] with rope_offset 0, or the rope columns
// 128..191 of per-head Q / K [B,S,H,192] -- that the reference leaves to its caller
// (reference/python/sources.json:2); it has no counterpart there.  rope_size a power of two
// up to 128; offset and width even.
void rope_apply_cuda(
    __hip_bfloat16* tensor,
    const int* positions,
    int batch_size,
    int sequence_length,
    int heads,
    int width,
    int rope_offset,
    int rope_size,
    float theta,
    hipStream_t stream = nullptr);

// The per-head projections either side of absorbed attention, which the reference leaves to its
// caller (reference/python/sources.json:2, "No ... model projections"); no counterpart there:
//     absorb     query_latent[t, h, c] = sum_d query_nope[t, h, d]  * w_uk[h, d, c]     d < 128, c < 512
//     un-absorb  output[t, h, d]       = sum_c output_latent[t, h, c] * w_uv[h, d, c]
// Both weights are [heads, 128, 512] BF16 (head h at w + h * weight_head_stride elements): the two
// halves of DeepSeek-V3's wkv_b viewed as [heads, 256, 512], stride 256 * 512.  Token t, head h of a
// tensor lies at base + t * token_stride + h * head_stride (elements), so the absorb can read the nope
// columns of a [B,S,H,192] query and write the latent columns of the packed [B,S,H,576] decode query
// directly.  BF16 in and out, FP32 accumulation.  All tensors aligned to 16 bytes, all strides multiples
// of 8 elements.
void mla_absorb_query_cuda(
    __hip_bfloat16* query_latent,
    const __hip_bfloat16* query_nope,
    const __hip_bfloat16* w_uk,
    long long tokens,
    int heads,
    long long query_nope_token_stride,
    long long query_nope_head_stride,
    long long query_latent_token_stride,
    long long query_latent_head_stride,
    long long weight_head_stride,
    hipStream_t stream = nullptr);

void mla_unabsorb_output_cuda(
    __hip_bfloat16* output,
    const __hip_bfloat16* output_latent,
    const __hip_bfloat16* w_uv,
    long long tokens,
    int heads,
    long long output_latent_token_stride,
    long long output_latent_head_stride,
    long long output_token_stride,
    long long output_head_stride,
    long long weight_head_stride,
    hipStream_t stream = nullptr);

}  // namespace dscuda

// ---- C ABI (libdscuda_mla_bench.so) ----------------------------------------
// Status 0 = ok, 1 = error; the message of the last error on the calling
// thread is returned by dscuda_mla_last_error() and stays valid until the next
// error on that thread.  Replaces reference benchmarks/bindings/mla_bridge.cpp
// symbols (mla_bridge.cu:12-73); argument order is identical.
extern "C" {

const char* dscuda_mla_last_error();  // mla_bridge.cu:12-14

int dscuda_mla_forward(  // mla_bridge.cu:16-31
    __hip_bfloat16* output, float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* query_rope,
    const __hip_bfloat16* latent, const __hip_bfloat16* key_rope,
    int batch, int sequence, int heads, int rank, int rope, float scale,
    hipStream_t stream);

int dscuda_mla_backward(  // mla_bridge.cu:33-51
    __hip_bfloat16* dquery, __hip_bfloat16* dquery_rope,
    __hip_bfloat16* dlatent, __hip_bfloat16* dkey_rope,
    const __hip_bfloat16* dout, const __hip_bfloat16* output, const float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* query_rope,
    const __hip_bfloat16* latent, const __hip_bfloat16* key_rope,
    int batch, int sequence, int heads, int rank, int rope, float scale,
    hipStream_t stream);

std::size_t dscuda_mla_workspace_elements(  // mla_bridge.cu:53-56
    int batch, int heads, int splits, int rank);

int dscuda_mla_decode(  // mla_bridge.cu:58-73
    __hip_bfloat16* output, float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* paged_cache,
    const int* block_table, const int* lengths, float* workspace,
    int batch, int heads, int rank, int rope, int page_size, int pages, int splits,
    float scale, hipStream_t stream);

// additive: the reusable decode plan (see dscuda::mla_decode_plan_cuda above)
std::size_t dscuda_mla_decode_plan_elements(int batch, int heads, int splits, int rank);

int dscuda_mla_decode_plan(
    int* plan, const int* lengths, int batch, int heads, int rank, int splits, hipStream_t stream);

int dscuda_mla_decode_planned(
    __hip_bfloat16* output, float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* paged_cache,
    const int* block_table, const int* lengths, float* workspace, int* plan,
    int batch, int heads, int rank, int rope, int page_size, int pages, int splits,
    float scale, hipStream_t stream);

// No counterpart in the reference: dscuda_mla_decode without the workspace argument, for
// callers that cannot allocate (see dscuda::mla_decode_forward_static above for the limit).
int dscuda_mla_decode_static(
    __hip_bfloat16* output, float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* paged_cache,
    const int* block_table, const int* lengths,
    int batch, int heads, int rank, int rope, int page_size, int pages, int splits,
    float scale, hipStream_t stream);

// additive (no counterpart in the reference)
int dscuda_mla_prefill_forward(
    __hip_bfloat16* output, float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* key, const __hip_bfloat16* value,
    int batch, int sequence, int heads, int qk_head_size, int v_head_size, float scale,
    hipStream_t stream);

std::size_t dscuda_mla_prefill_backward_workspace_elements(
    int batch, int sequence, int heads, int qk_head_size, int v_head_size);

// additive (no counterpart in the reference): tuning knobs, see the dscuda:: functions of the same names above
void dscuda_mla_prefill_backward_set_workspace_limit(std::size_t bytes);
void dscuda_mla_backward_set_key_interval_tiles(int tiles);

int dscuda_mla_prefill_backward(
    __hip_bfloat16* dquery, __hip_bfloat16* dkey, __hip_bfloat16* dvalue,
    const __hip_bfloat16* dout, const __hip_bfloat16* output, const float* lse,
    const __hip_bfloat16* query, const __hip_bfloat16* key, const __hip_bfloat16* value,
    float* workspace,
    int batch, int sequence, int heads, int qk_head_size, int v_head_size, float scale,
    hipStream_t stream);

// additive (no counterpart in the reference): see dscuda::rope_apply_cuda above; errors through dscuda_mla_last_error
int dscuda_rope_apply(
    __hip_bfloat16* tensor, const int* positions,
    int batch, int sequence, int heads, int width, int rope_offset, int rope_size, float theta,
    hipStream_t stream);

// additive (no counterpart in the reference): see dscuda::mla_absorb_query_cuda / mla_unabsorb_output_cuda above
int dscuda_mla_absorb_query(
    __hip_bfloat16* query_latent, const __hip_bfloat16* query_nope, const __hip_bfloat16* w_uk,
    long long tokens, int heads,
    long long query_nope_token_stride, long long query_nope_head_stride,
    long long query_latent_token_stride, long long query_latent_head_stride,
    long long weight_head_stride, hipStream_t stream);

int dscuda_mla_unabsorb_output(
    __hip_bfloat16* output, const __hip_bfloat16* output_latent, const __hip_bfloat16* w_uv,
    long long tokens, int heads,
    long long output_latent_token_stride, long long output_latent_head_stride,
    long long output_token_stride, long long output_head_stride,
    long long weight_head_stride, hipStream_t stream);

}  // extern "C"
