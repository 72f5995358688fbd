// Entry points and C-ABI bridge of the MLA kernels.
//
// The dscuda:: functions validate their arguments before any runtime call
// (the reference's check_shape, kernels/attention/mla/sm89.cu:20-24, throws
// std::invalid_argument("MLA requires C=512 and RoPE=64") first thing, which
// makes the error path testable on a host without a GPU) and then hand over to
// the kernel translation units.  The extern "C" wrappers follow
// benchmarks/bindings/mla_bridge.cu:12-73: status 0 / 1 and a thread-local
// message, exceptions never cross the C boundary.
#include "../../include/mla.h"

#include "attn_kernels.h"
#include "hip_common.h"

#include <exception>
#include <mutex>
#include <stdexcept>
#include <string>

namespace dscuda {
namespace {

void check_shape(int kv_rank, int rope_size) {
    if (kv_rank != MLA_KV_RANK || rope_size != MLA_ROPE_SIZE) {
        throw std::invalid_argument("MLA requires C=512 and RoPE=64");
    }
}

void check_positive(const char* what, int batch_size, int tokens, int heads) {
    if (batch_size <= 0 || tokens <= 0 || heads <= 0) {
        throw std::invalid_argument(std::string(what) + " requires positive batch, sequence and head counts");
    }
}

// Workspace of mla_decode_forward_static: one array per GPU, part of the loaded code
// object, so it exists from module load to process exit and no call ever allocates.
// In host code the array's name only stands for the symbol; the device address is
// looked up once per device and every use below goes through that pointer.
__device__ __align__(256) unsigned char static_decode_scratch[MLA_DECODE_STATIC_SCRATCH_BYTES];

float* static_decode_scratch_of_current_device() {
    static std::mutex guard;
    static void* address_of_device[hip_common::MAX_DEVICES] = {};
    const int device = hip_common::current_device();
    std::lock_guard<std::mutex> lock(guard);
    if (address_of_device[device] == nullptr) {
        void* address = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(static_decode_scratch)));
        if (address == nullptr) {
            throw std::runtime_error("MLA decode (static workspace): the workspace symbol has no device address");
        }
        address_of_device[device] = address;
    }
    return static_cast<float*>(address_of_device[device]);
}

void check_prefill_heads(int qk_head_size, int v_head_size) {
    const bool ok = (qk_head_size == 192 && v_head_size == 128) || (qk_head_size == 128 && v_head_size == 128) ||
                    (qk_head_size == 64 && v_head_size == 64);
    if (!ok) {
        throw std::invalid_argument("MLA prefill requires (d_qk,d_v) in {(192,128),(128,128),(64,64)}");
    }
}

}  // namespace

void mla_compressed_attention_forward_cuda(__hip_bfloat16* output, float* logsumexp,
                                           const __hip_bfloat16* query_latent, const __hip_bfloat16* query_rope,
                                           const __hip_bfloat16* kv_latent, const __hip_bfloat16* key_rope,
                                           int batch_size, int sequence_length, int heads, int kv_rank, int rope_size,
                                           float scale, hipStream_t stream) {
    check_shape(kv_rank, rope_size);
    check_positive("MLA forward", batch_size, sequence_length, heads);
    mla_absorbed_forward_dispatch(output, logsumexp, query_latent, query_rope, kv_latent, key_rope, batch_size,
                                  sequence_length, heads, scale, stream);
}

void mla_compressed_attention_backward_cuda(
    __hip_bfloat16* query_latent_gradient, __hip_bfloat16* query_rope_gradient, __hip_bfloat16* kv_latent_gradient,
    __hip_bfloat16* key_rope_gradient, const __hip_bfloat16* output_gradient, const __hip_bfloat16* output,
    const float* logsumexp, const __hip_bfloat16* query_latent, const __hip_bfloat16* query_rope,
    const __hip_bfloat16* kv_latent, const __hip_bfloat16* key_rope, int batch_size, int sequence_length, int heads,
    int kv_rank, int rope_size, float scale, hipStream_t stream) {
    check_shape(kv_rank, rope_size);
    check_positive("MLA backward", batch_size, sequence_length, heads);
    mla_absorbed_backward_dispatch(query_latent_gradient, query_rope_gradient, kv_latent_gradient, key_rope_gradient,
                                   output_gradient, output, logsumexp, query_latent, query_rope, kv_latent, key_rope,
                                   batch_size, sequence_length, heads, scale, stream);
}

std::size_t mla_decode_workspace_elements(int batch_size, int heads, int splits, int kv_rank) {
    // reference kernels/attention/mla/sm89.cu:539-541
    return static_cast<std::size_t>(batch_size) * heads * splits * (kv_rank + 2);
}

void mla_decode_forward_cuda(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                             const __hip_bfloat16* paged_kv_cache, const int* block_table, const int* cache_lengths,
                             float* workspace, int batch_size, int heads, int kv_rank, int rope_size, int page_size,
                             int pages_per_sequence, int splits, float scale, hipStream_t stream) {
    check_shape(kv_rank, rope_size);
    if (batch_size <= 0 || heads <= 0 || page_size <= 0 || pages_per_sequence <= 0 || splits <= 0) {
        throw std::invalid_argument(
            "MLA decode requires positive batch, head, page_size, pages_per_sequence and splits");
    }
    mla_decode_dispatch(output, logsumexp, query, paged_kv_cache, block_table, cache_lengths, workspace, nullptr,
                        batch_size, heads, page_size, pages_per_sequence, splits, scale, stream);
}

std::size_t mla_decode_plan_elements(int batch_size, int heads, int splits, int kv_rank) {
    if (batch_size <= 0 || heads <= 0 || splits <= 0 || kv_rank != MLA_KV_RANK) {
        return 0;
    }
    return dscuda::mla_decode_plan_elements(batch_size, heads, splits);
}

void mla_decode_plan_cuda(int* plan, const int* cache_lengths, int batch_size, int heads, int kv_rank, int splits,
                          hipStream_t stream) {
    check_shape(kv_rank, MLA_ROPE_SIZE);
    if (batch_size <= 0 || heads <= 0 || splits <= 0) {
        throw std::invalid_argument("MLA decode plan requires positive batch, head and split counts");
    }
    if (plan == nullptr || cache_lengths == nullptr) {
        throw std::invalid_argument("MLA decode plan requires a plan buffer and the cache lengths");
    }
    mla_decode_plan_dispatch(plan, cache_lengths, batch_size, heads, splits, stream);
}

void mla_decode_forward_planned_cuda(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                                     const __hip_bfloat16* paged_kv_cache, const int* block_table,
                                     const int* cache_lengths, float* workspace, int* plan, int batch_size, int heads,
                                     int kv_rank, int rope_size, int page_size, int pages_per_sequence, int splits,
                                     float scale, hipStream_t stream) {
    check_shape(kv_rank, rope_size);
    if (batch_size <= 0 || heads <= 0 || page_size <= 0 || pages_per_sequence <= 0 || splits <= 0) {
        throw std::invalid_argument(
            "MLA decode requires positive batch, head, page_size, pages_per_sequence and splits");
    }
    if (plan == nullptr) {
        throw std::invalid_argument("MLA decode (planned) requires the plan written by mla_decode_plan_cuda");
    }
    mla_decode_dispatch(output, logsumexp, query, paged_kv_cache, block_table, cache_lengths, workspace, plan,
                        batch_size, heads, page_size, pages_per_sequence, splits, scale, stream);
}

void mla_decode_forward_static(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                               const __hip_bfloat16* paged_kv_cache, const int* block_table, const int* cache_lengths,
                               int batch_size, int heads, int kv_rank, int rope_size, int page_size,
                               int pages_per_sequence, int splits, float scale, hipStream_t stream) {
    check_shape(kv_rank, rope_size);
    if (batch_size <= 0 || heads <= 0 || page_size <= 0 || pages_per_sequence <= 0 || splits <= 0) {
        throw std::invalid_argument(
            "MLA decode requires positive batch, head, page_size, pages_per_sequence and splits");
    }
    const std::size_t needed = mla_decode_workspace_elements(batch_size, heads, splits, kv_rank) * sizeof(float);
    if (needed > MLA_DECODE_STATIC_SCRATCH_BYTES) {
        throw std::invalid_argument(
            "MLA decode (static workspace): batch*heads*splits*(rank+2) floats = " + std::to_string(needed) +
            " bytes exceed the built-in workspace of " + std::to_string(MLA_DECODE_STATIC_SCRATCH_BYTES) +
            " bytes; lower splits or call the variant that takes a caller workspace");
    }
    float* workspace = static_decode_scratch_of_current_device();
    mla_decode_dispatch(output, logsumexp, query, paged_kv_cache, block_table, cache_lengths, workspace, nullptr,
                        batch_size, heads, page_size, pages_per_sequence, splits, scale, stream);
}

void mla_prefill_forward_cuda(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                              const __hip_bfloat16* key, const __hip_bfloat16* value, int batch_size,
                              int sequence_length, int heads, int qk_head_size, int v_head_size, float scale,
                              hipStream_t stream) {
    check_prefill_heads(qk_head_size, v_head_size);
    check_positive("MLA prefill forward", batch_size, sequence_length, heads);
    attention_forward_dispatch(output, logsumexp, query, key, value, batch_size, sequence_length, heads, heads,
                               qk_head_size, v_head_size, scale, stream);
}

std::size_t mla_prefill_backward_workspace_elements(int batch_size, int sequence_length, int heads,
                                                    int /*qk_head_size*/, int /*v_head_size*/) {
    if (batch_size <= 0 || sequence_length <= 0 || heads <= 0) {
        return 0;
    }
    return attention_backward_workspace_elements(batch_size, sequence_length, heads, heads);
}

void mla_prefill_backward_set_workspace_limit(std::size_t bytes) {
    attention_backward_set_workspace_limit(bytes);
}

void mla_backward_set_key_interval_tiles(int tiles) {
    mla_absorbed_backward_set_key_interval_tiles(tiles);
}

void mla_prefill_backward_cuda(__hip_bfloat16* query_gradient, __hip_bfloat16* key_gradient,
                               __hip_bfloat16* value_gradient, const __hip_bfloat16* output_gradient,
                               const __hip_bfloat16* output, const float* logsumexp, const __hip_bfloat16* query,
                               const __hip_bfloat16* key, const __hip_bfloat16* value, float* workspace,
                               int batch_size, int sequence_length, int heads, int qk_head_size, int v_head_size,
                               float scale, hipStream_t stream) {
    check_prefill_heads(qk_head_size, v_head_size);
    check_positive("MLA prefill backward", batch_size, sequence_length, heads);
    if (workspace == nullptr) {
        throw std::invalid_argument("MLA prefill backward requires a workspace");
    }
    attention_backward_dispatch(query_gradient, key_gradient, value_gradient, output_gradient, output, logsumexp, query,
                                key, value, workspace, batch_size, sequence_length, heads, heads, qk_head_size,
                                v_head_size, scale, stream);
}

void rope_apply_cuda(__hip_bfloat16* tensor, const int* positions, int batch_size, int sequence_length, int heads,
                     int width, int rope_offset, int rope_size, float theta, hipStream_t stream) {
    rope_apply_dispatch(tensor, positions, batch_size, sequence_length, heads, width, rope_offset, rope_size, theta, stream);
}

void mla_absorb_query_cuda(__hip_bfloat16* query_latent, const __hip_bfloat16* query_nope, const __hip_bfloat16* w_uk,
                           long long tokens, int heads, long long query_nope_token_stride,
                           long long query_nope_head_stride, long long query_latent_token_stride,
                           long long query_latent_head_stride, long long weight_head_stride, hipStream_t stream) {
    mla_absorb_query_dispatch(query_latent, query_nope, w_uk, tokens, heads, query_nope_token_stride,
                              query_nope_head_stride, query_latent_token_stride, query_latent_head_stride,
                              weight_head_stride, stream);
}

void mla_unabsorb_output_cuda(__hip_bfloat16* output, const __hip_bfloat16* output_latent, const __hip_bfloat16* w_uv,
                              long long tokens, int heads, long long output_latent_token_stride,
                              long long output_latent_head_stride, long long output_token_stride,
                              long long output_head_stride, long long weight_head_stride, hipStream_t stream) {
    mla_unabsorb_output_dispatch(output, output_latent, w_uv, tokens, heads, output_latent_token_stride,
                                 output_latent_head_stride, output_token_stride, output_head_stride,
                                 weight_head_stride, stream);
}

}  // namespace dscuda

namespace {
thread_local std::string last_error;

template <typename Call>
int guarded(Call&& call) {
    try {
        call();
        return 0;
    } catch (const std::exception& error) {
        last_error = error.what();
        return 1;
    }
}
}  // namespace

extern "C" const char* dscuda_mla_last_error() {
    return last_error.c_str();
}

extern "C" int dscuda_mla_forward(__hip_bfloat16* output, float* lse, const __hip_bfloat16* query,
                                  const __hip_bfloat16* query_rope, const __hip_bfloat16* latent,
                                  const __hip_bfloat16* key_rope, int batch, int sequence, int heads, int rank,
                                  int rope, float scale, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_compressed_attention_forward_cuda(output, lse, query, query_rope, latent, key_rope, batch,
                                                      sequence, heads, rank, rope, scale, stream);
    });
}

extern "C" int dscuda_mla_backward(__hip_bfloat16* dquery, __hip_bfloat16* dquery_rope, __hip_bfloat16* dlatent,
                                   __hip_bfloat16* dkey_rope, const __hip_bfloat16* dout,
                                   const __hip_bfloat16* output, const float* lse, const __hip_bfloat16* query,
                                   const __hip_bfloat16* query_rope, const __hip_bfloat16* latent,
                                   const __hip_bfloat16* key_rope, int batch, int sequence, int heads, int rank,
                                   int rope, float scale, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_compressed_attention_backward_cuda(dquery, dquery_rope, dlatent, dkey_rope, dout, output, lse,
                                                       query, query_rope, latent, key_rope, batch, sequence, heads,
                                                       rank, rope, scale, stream);
    });
}

extern "C" std::size_t dscuda_mla_workspace_elements(int batch, int heads, int splits, int rank) {
    std::size_t elements = 0;
    guarded([&] { elements = dscuda::mla_decode_workspace_elements(batch, heads, splits, rank); });
    return elements;
}

extern "C" int dscuda_mla_decode(__hip_bfloat16* output, float* lse, const __hip_bfloat16* query,
                                 const __hip_bfloat16* paged_cache, const int* block_table, const int* lengths,
                                 float* workspace, int batch, int heads, int rank, int rope, int page_size, int pages,
                                 int splits, float scale, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_decode_forward_cuda(output, lse, query, paged_cache, block_table, lengths, workspace, batch,
                                        heads, rank, rope, page_size, pages, splits, scale, stream);
    });
}

extern "C" std::size_t dscuda_mla_decode_plan_elements(int batch, int heads, int splits, int rank) {
    std::size_t elements = 0;
    guarded([&] { elements = dscuda::mla_decode_plan_elements(batch, heads, splits, rank); });
    return elements;   // 0 with the message set when the arguments admit no plan
}

extern "C" int dscuda_mla_decode_plan(int* plan, const int* lengths, int batch, int heads, int rank, int splits,
                                      hipStream_t stream) {
    return guarded([&] { dscuda::mla_decode_plan_cuda(plan, lengths, batch, heads, rank, splits, stream); });
}

extern "C" int dscuda_mla_decode_planned(__hip_bfloat16* output, float* lse, const __hip_bfloat16* query,
                                         const __hip_bfloat16* paged_cache, const int* block_table, const int* lengths,
                                         float* workspace, int* plan, int batch, int heads, int rank, int rope,
                                         int page_size, int pages, int splits, float scale, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_decode_forward_planned_cuda(output, lse, query, paged_cache, block_table, lengths, workspace, plan,
                                                batch, heads, rank, rope, page_size, pages, splits, scale, stream);
    });
}

extern "C" int dscuda_mla_decode_static(__hip_bfloat16* output, float* lse, const __hip_bfloat16* query,
                                        const __hip_bfloat16* paged_cache, const int* block_table,
                                        const int* lengths, int batch, int heads, int rank, int rope, int page_size,
                                        int pages, int splits, float scale, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_decode_forward_static(output, lse, query, paged_cache, block_table, lengths, batch, heads, rank,
                                          rope, page_size, pages, splits, scale, stream);
    });
}

extern "C" int dscuda_mla_prefill_forward(__hip_bfloat16* output, float* lse, const __hip_bfloat16* query,
                                          const __hip_bfloat16* key, const __hip_bfloat16* value, int batch,
                                          int sequence, int heads, int qk_head_size, int v_head_size, float scale,
                                          hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_prefill_forward_cuda(output, lse, query, key, value, batch, sequence, heads, qk_head_size,
                                         v_head_size, scale, stream);
    });
}

extern "C" std::size_t dscuda_mla_prefill_backward_workspace_elements(int batch, int sequence, int heads,
                                                                      int qk_head_size, int v_head_size) {
    std::size_t elements = 0;
    guarded([&] {
        elements = dscuda::mla_prefill_backward_workspace_elements(batch, sequence, heads, qk_head_size, v_head_size);
    });
    return elements;
}

extern "C" void dscuda_mla_prefill_backward_set_workspace_limit(std::size_t bytes) {
    dscuda::mla_prefill_backward_set_workspace_limit(bytes);
}

extern "C" void dscuda_mla_backward_set_key_interval_tiles(int tiles) {
    dscuda::mla_backward_set_key_interval_tiles(tiles);
}

extern "C" int dscuda_mla_prefill_backward(__hip_bfloat16* dquery, __hip_bfloat16* dkey, __hip_bfloat16* dvalue,
                                           const __hip_bfloat16* dout, const __hip_bfloat16* output, const float* lse,
                                           const __hip_bfloat16* query, const __hip_bfloat16* key,
                                           const __hip_bfloat16* value, float* workspace, int batch, int sequence,
                                           int heads, int qk_head_size, int v_head_size, float scale,
                                           hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_prefill_backward_cuda(dquery, dkey, dvalue, dout, output, lse, query, key, value, workspace,
                                          batch, sequence, heads, qk_head_size, v_head_size, scale, stream);
    });
}

extern "C" int dscuda_rope_apply(__hip_bfloat16* tensor, const int* positions, int batch, int sequence, int heads,
                                 int width, int rope_offset, int rope_size, float theta, hipStream_t stream) {
    return guarded([&] {
        dscuda::rope_apply_cuda(tensor, positions, batch, sequence, heads, width, rope_offset, rope_size, theta, stream);
    });
}

extern "C" int dscuda_mla_absorb_query(__hip_bfloat16* query_latent, const __hip_bfloat16* query_nope,
                                       const __hip_bfloat16* w_uk, long long tokens, int heads,
                                       long long query_nope_token_stride, long long query_nope_head_stride,
                                       long long query_latent_token_stride, long long query_latent_head_stride,
                                       long long weight_head_stride, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_absorb_query_cuda(query_latent, query_nope, w_uk, tokens, heads, query_nope_token_stride,
                                      query_nope_head_stride, query_latent_token_stride, query_latent_head_stride,
                                      weight_head_stride, stream);
    });
}

extern "C" int dscuda_mla_unabsorb_output(__hip_bfloat16* output, const __hip_bfloat16* output_latent,
                                          const __hip_bfloat16* w_uv, long long tokens, int heads,
                                          long long output_latent_token_stride, long long output_latent_head_stride,
                                          long long output_token_stride, long long output_head_stride,
                                          long long weight_head_stride, hipStream_t stream) {
    return guarded([&] {
        dscuda::mla_unabsorb_output_cuda(output, output_latent, w_uv, tokens, heads, output_latent_token_stride,
                                         output_latent_head_stride, output_token_stride, output_head_stride,
                                         weight_head_stride, stream);
    });
}
