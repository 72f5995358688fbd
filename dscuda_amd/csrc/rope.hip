// Rotary position embedding applied in place to a slice of the last dimension of a
// [B, S, H, W] bf16 tensor: the step that precedes the attention kernels in an MLA
// layer (the rope parts of Q and K) and that the reference leaves to its caller
// (reference/python/sources.json:2 lists "model projections" and position encoding
// among the things it does not contain).
//
// Convention: interleaved pairs.  Within the slice of `rope` columns, columns
// (2i, 2i + 1) form pair i, rotated by the angle position * theta^(-2i / rope):
//     x'[2i]     = x[2i] * cos - x[2i + 1] * sin
//     x'[2i + 1] = x[2i] * sin + x[2i + 1] * cos
// with position = s (+ positions[b] when a per-sequence start is given, as for the one
// new token of a decode step).  Frequencies and angles are formed in double precision
// and the sine and cosine rounded to fp32 once, the products and the sum each rounded to
// fp32 without fusing, the result rounded to bf16: the same sequence of roundings as
// forming the rotation with fp32 tensors on the host.
//
// Layout on the chip: one wave per (batch, position).  A lane owns pair lane % (rope/2)
// and computes its sine and cosine once; the 64 / (rope/2) groups of lanes then walk the
// heads in turn, so every access of a group is one contiguous run of 2 * rope bytes.
// The kernel moves 4 * rope bytes per (b, s, h) and is bound by memory.

#include "attn_kernels.h"
#include "hip_common.h"

#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <string>

namespace dscuda {
namespace {

constexpr int ROPE_THREADS = 256;
constexpr int ROPE_ROWS = ROPE_THREADS / 64;   // (batch, position) rows per workgroup

__global__ __launch_bounds__(ROPE_THREADS) void rope_apply_kernel(bf16_t* __restrict__ tensor,
                                                                  const int* __restrict__ positions, long long rows,
                                                                  int sequence_length, int heads, int width,
                                                                  int rope_offset, int rope, double log2_theta) {
    const long long row = (long long)blockIdx.x * ROPE_ROWS + threadIdx.x / 64;
    if (row >= rows) return;
    const int lane = threadIdx.x % 64;
    const int pairs = rope / 2;            // a power of two, at most 64
    const int pair = lane % pairs;
    const int group = lane / pairs;
    const int groups = 64 / pairs;
    const long long b = row / sequence_length;
    const int s = (int)(row % sequence_length);
    const int position = s + (positions ? positions[b] : 0);
    const double frequency = exp2(-log2_theta * (2.0 * pair / rope));
    const double angle = (double)position * frequency;
    const float cosine = (float)cos(angle);
    const float sine = (float)sin(angle);
    unsigned* base = reinterpret_cast<unsigned*>(tensor + (size_t)row * heads * width + rope_offset) + pair;
    for (int h = group; h < heads; h += groups) {
        unsigned* target = base + (size_t)h * (width / 2);
        const unsigned bits = *target;
        const float even = __uint_as_float(bits << 16);
        const float odd = __uint_as_float(bits & 0xffff0000u);
        const float rotated_even = __fsub_rn(__fmul_rn(even, cosine), __fmul_rn(odd, sine));
        const float rotated_odd = __fadd_rn(__fmul_rn(even, sine), __fmul_rn(odd, cosine));
        *target = pack_bf16(rotated_even, rotated_odd);
    }
}

}  // namespace

void rope_apply_dispatch(bf16_t* tensor, const int* positions, int batch_size, int sequence_length, int heads, int width,
                         int rope_offset, int rope_size, float theta, hipStream_t stream) {
    if (batch_size <= 0 || sequence_length <= 0 || heads <= 0) {
        throw std::invalid_argument("rope: batch, sequence length and heads must be positive");
    }
    const bool power_of_two = rope_size >= 2 && (rope_size & (rope_size - 1)) == 0;
    if (!power_of_two || rope_size > 128) {
        throw std::invalid_argument("rope: the rotated slice must be 2, 4, ..., 128 columns wide, got " +
                                    std::to_string(rope_size));
    }
    // pairs are moved as 32-bit words: the slice must start at an even column of rows of even width
    if (width <= 0 || width % 2 != 0 || rope_offset < 0 || rope_offset % 2 != 0 || rope_offset + rope_size > width) {
        throw std::invalid_argument("rope: columns " + std::to_string(rope_offset) + ".." +
                                    std::to_string(rope_offset + rope_size) + " do not fit rows of " +
                                    std::to_string(width) + " columns (even offset and width required)");
    }
    if (!(theta > 0.f)) {
        throw std::invalid_argument("rope: theta must be positive");
    }
    if (tensor == nullptr || reinterpret_cast<uintptr_t>(tensor) % 4 != 0) {
        throw std::invalid_argument("rope: the tensor must be a non-null pointer aligned to 4 bytes");
    }
    const long long rows = (long long)batch_size * sequence_length;
    const long long blocks = (rows + ROPE_ROWS - 1) / ROPE_ROWS;
    if (blocks > 0x7fffffffLL) {
        throw std::invalid_argument("rope: batch * sequence length exceeds the grid limit");
    }
    hipLaunchKernelGGL(rope_apply_kernel, dim3((unsigned)blocks), dim3(ROPE_THREADS), 0, stream, tensor, positions, rows,
                       sequence_length, heads, width, rope_offset, rope_size, std::log2((double)theta));
    HIP_CHECK(hipGetLastError());
}

}  // namespace dscuda
