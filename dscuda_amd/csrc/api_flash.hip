// Entry point and C-ABI bridge of the causal flash-attention forward.
//
// flash_attention_forward_cuda validates like the reference's host wrapper
// (kernels/attention/flash_attention/sm89_forward.cu:222-235,
// sm89_common.cuh:172-176) -- same exception type, same messages apart from
// the wider head-size rule -- and then launches the gfx950 kernel.  The
// extern "C" wrappers follow benchmarks/bindings/flash_attention_bridge.cu:
// exceptions never cross the C boundary, they become status 1 plus a
// thread-local message.
#include "../../include/flash_attention.h"

#include "attn_kernels.h"
#include "hip_common.h"

#include <exception>
#include <stdexcept>
#include <string>

namespace dscuda {

void flash_attention_forward_cuda(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                                  const __hip_bfloat16* key, const __hip_bfloat16* value, int batch_size,
                                  int sequence_length, int query_heads, int key_value_heads, int head_size,
                                  float scale, hipStream_t stream) {
    if (head_size != 64 && head_size != 128) {
        throw std::runtime_error("flash attention requires head_size = 64 or 128");
    }
    if (sequence_length <= 0 || sequence_length % 64 != 0) {
        throw std::runtime_error("flash attention requires T to be a positive multiple of 64");
    }
    if (query_heads <= 0 || key_value_heads <= 0 || query_heads % key_value_heads != 0) {
        throw std::runtime_error("flash attention requires query_heads to be divisible by key_value_heads");
    }
    if (batch_size <= 0) {
        throw std::runtime_error("flash attention requires a positive batch size");
    }
    attention_forward_dispatch(output, logsumexp, query, key, value, batch_size, sequence_length, query_heads,
                               key_value_heads, head_size, head_size, scale, stream);
}

namespace {
void check_flash_backward_shape(int batch_size, int sequence_length, int query_heads, int key_value_heads, int head_size) {
    if (head_size != 64 && head_size != 128) {
        throw std::runtime_error("flash attention requires head_size = 64 or 128");
    }
    if (sequence_length <= 0) {
        throw std::runtime_error("flash attention backward requires a positive T");
    }
    if (query_heads <= 0 || key_value_heads <= 0 || query_heads % key_value_heads != 0) {
        throw std::runtime_error("flash attention requires query_heads to be divisible by key_value_heads");
    }
    if (batch_size <= 0) {
        throw std::runtime_error("flash attention requires a positive batch size");
    }
}
}  // namespace

std::size_t flash_attention_backward_workspace_elements(int batch_size, int sequence_length, int query_heads,
                                                        int key_value_heads, int head_size) {
    if (batch_size <= 0 || sequence_length <= 0 || query_heads <= 0 || key_value_heads <= 0 ||
        query_heads % key_value_heads != 0 || (head_size != 64 && head_size != 128)) {
        return 0;
    }
    return attention_backward_workspace_elements(batch_size, sequence_length, query_heads, key_value_heads);
}

void flash_attention_backward_set_workspace_limit(std::size_t bytes) {
    attention_backward_set_workspace_limit(bytes);
}

void flash_attention_backward_cuda(__hip_bfloat16* query_gradient, __hip_bfloat16* key_gradient,
                                   __hip_bfloat16* value_gradient, const __hip_bfloat16* output_gradient,
                                   const __hip_bfloat16* output, const float* logsumexp, const __hip_bfloat16* query,
                                   const __hip_bfloat16* key, const __hip_bfloat16* value, float* workspace,
                                   int batch_size, int sequence_length, int query_heads, int key_value_heads,
                                   int head_size, float scale, hipStream_t stream) {
    check_flash_backward_shape(batch_size, sequence_length, query_heads, key_value_heads, head_size);
    if (workspace == nullptr) {
        throw std::runtime_error("flash attention backward requires a workspace");
    }
    attention_backward_dispatch(query_gradient, key_gradient, value_gradient, output_gradient, output, logsumexp, query,
                                key, value, workspace, batch_size, sequence_length, query_heads, key_value_heads,
                                head_size, head_size, scale, stream);
}

}  // namespace dscuda

namespace {
thread_local std::string last_error;
}

extern "C" const char* dscuda_flash_last_error() {
    return last_error.c_str();
}

extern "C" int dscuda_flash_forward(__hip_bfloat16* output, float* logsumexp, const __hip_bfloat16* query,
                                    const __hip_bfloat16* key, const __hip_bfloat16* value, int batch, int sequence,
                                    int query_heads, int key_value_heads, int dimension, float scale,
                                    hipStream_t stream) {
    try {
        dscuda::flash_attention_forward_cuda(output, logsumexp, query, key, value, batch, sequence, query_heads,
                                             key_value_heads, dimension, scale, stream);
        return 0;
    } catch (const std::exception& error) {
        last_error = error.what();
        return 1;
    }
}

extern "C" std::size_t dscuda_flash_backward_workspace_elements(int batch, int sequence, int query_heads,
                                                                int key_value_heads, int dimension) {
    try {
        return dscuda::flash_attention_backward_workspace_elements(batch, sequence, query_heads, key_value_heads,
                                                                   dimension);
    } catch (const std::exception& error) {
        last_error = error.what();
        return 0;
    }
}

extern "C" void dscuda_flash_backward_set_workspace_limit(std::size_t bytes) {
    dscuda::flash_attention_backward_set_workspace_limit(bytes);
}

extern "C" int dscuda_flash_backward(__hip_bfloat16* dquery, __hip_bfloat16* dkey, __hip_bfloat16* dvalue,
                                     const __hip_bfloat16* dout, const __hip_bfloat16* output, const float* logsumexp,
                                     const __hip_bfloat16* query, const __hip_bfloat16* key, const __hip_bfloat16* value,
                                     float* workspace, int batch, int sequence, int query_heads, int key_value_heads,
                                     int dimension, float scale, hipStream_t stream) {
    try {
        dscuda::flash_attention_backward_cuda(dquery, dkey, dvalue, dout, output, logsumexp, query, key, value, workspace,
                                              batch, sequence, query_heads, key_value_heads, dimension, scale, stream);
        return 0;
    } catch (const std::exception& error) {
        last_error = error.what();
        return 1;
    }
}
