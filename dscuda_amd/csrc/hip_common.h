// Shared host/device helpers for the gfx950 attention kernels.
//
// Host side: HIP_CHECK turns a failing runtime call into a std::runtime_error
// carrying file:line and the evaluated expression, the same contract as the
// reference's CUDA_CHECK (include/cuda_common.h:10-25,
// kernels/common/cuda_common.cu:24-32).  The C-ABI bridges catch it and hand
// the text back through dscuda_*_last_error().
//
// Device side: vector typedefs for the bf16 MFMA builtins and the few
// cross-lane / conversion primitives every kernel uses.  Lane layouts of the
// two MFMA shapes used here (wave64, l = lane id):
//
//   mfma_f32_32x32x16_bf16   A: row l%32, k = 8*(l/32)+j      (8 bf16 / lane)
//                            B: col l%32, k = 8*(l/32)+j
//                            C: col l%32, row 8*(i/4)+4*(l/32)+i%4, i = 0..15
//   mfma_f32_16x16x32_bf16   A: row l%16, k = 8*(l/16)+j
//                            B: col l%16, k = 8*(l/16)+j
//                            C: col l%16, row 4*(l/16)+i, i = 0..3
//
// Because the contraction index only has to agree between A and B, any
// permutation of k that both operands share gives the same product; the
// kernels use that to feed a C-layout tile straight back in as a B operand.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>

namespace dscuda {

inline void hip_check(hipError_t result, const char* expression, const char* file, int line) {
    if (result == hipSuccess) {
        return;
    }
    std::ostringstream message;
    message << "HIP failure at " << file << ':' << line << " while evaluating " << expression << ": "
            << hipGetErrorString(result);
    throw std::runtime_error(message.str());
}

#define HIP_CHECK(expression) ::dscuda::hip_check((expression), #expression, __FILE__, __LINE__)

using bf16_t = __hip_bfloat16;

// What the host side remembers per device: attributes of a kernel (hipFuncSetAttribute acts on
// the current device's copy of the function) and device properties are set or asked once for
// each device a thread makes current, not once per thread or per process.
namespace hip_common {

constexpr int MAX_DEVICES = 64;

inline int current_device() {
    int device = 0;
    HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= MAX_DEVICES) {
        throw std::runtime_error("device index " + std::to_string(device) + " is beyond the " +
                                 std::to_string(MAX_DEVICES) + " devices this library keeps state for");
    }
    return device;
}

// Runs `prepare` the first time it is asked to on each device.  Two threads may both run it for
// the same device (the preparation is idempotent); none skips it before it has completed once.
class OncePerDevice {
public:
    template <typename Prepare>
    void run(Prepare&& prepare) {
        const int device = current_device();
        if (!done_[device].load(std::memory_order_acquire)) {
            prepare();
            done_[device].store(true, std::memory_order_release);
        }
    }

private:
    std::atomic<bool> done_[MAX_DEVICES] = {};
};

// Compute units of the current device, asked once per device.
inline int compute_units_of_current_device() {
    static std::atomic<int> units_of_device[MAX_DEVICES] = {};
    const int device = current_device();
    int units = units_of_device[device].load(std::memory_order_relaxed);
    if (units == 0) {
        HIP_CHECK(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device));
        units_of_device[device].store(units, std::memory_order_relaxed);
    }
    return units;
}

}  // namespace hip_common

#if defined(__HIP_DEVICE_COMPILE__) || defined(__HIPCC__)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

// Value held by the lane 32 places away, combined with the lane's own by a
// symmetric op.  v_permlane32_swap exchanges the upper half of its first
// operand with the lower half of its second, so feeding the same register to
// both leaves {own, other} (in one order or the other) in the two results.
__device__ __forceinline__ float half_wave_max(float value) {
    auto swapped = __builtin_amdgcn_permlane32_swap(__float_as_uint(value), __float_as_uint(value), false, false);
    return fmaxf(__uint_as_float(swapped[0]), __uint_as_float(swapped[1]));
}

__device__ __forceinline__ float half_wave_sum(float value) {
    auto swapped = __builtin_amdgcn_permlane32_swap(__float_as_uint(value), __float_as_uint(value), false, false);
    return __uint_as_float(swapped[0]) + __uint_as_float(swapped[1]);
}

// Two fp32 -> packed bf16 (round to nearest even, one v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float low, float high) {
    f32x2 pair = {low, high};
    bf16x2 packed = __builtin_convertvector(pair, bf16x2);
    return __builtin_bit_cast(uint32_t, packed);
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}

// ---- direct global -> LDS loads and the synchronisation that goes with them ----
//
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight
// into LDS at (M0 base) + 16 * lane; a wave instruction fills 1 KB of
// consecutive LDS.  The loads are issued as asm so that the compiler's
// wait-count bookkeeping does not see an LDS writer: it would otherwise drain
// every outstanding load before each LDS read of the tile being consumed and
// serialise the prefetch.  Arrival is ordered by hand: wait_vector_memory
// (per wave) followed by workgroup_barrier (all waves).

typedef __attribute__((address_space(3))) void* lds_pointer;

__device__ __forceinline__ unsigned lds_offset_of(const void* pointer) {
    return (unsigned)(uintptr_t)(lds_pointer)pointer;
}

// source = per-lane 64-bit address; lds_base wave-uniform
__device__ __forceinline__ void direct_load_16(const void* source, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(source), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory", "m0");
}

// source = uniform 64-bit base + per-lane 32-bit byte offset; lds_base wave-uniform
__device__ __forceinline__ void direct_load_16_offset(const void* uniform_base, unsigned byte_offset, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(byte_offset), "s"(uniform_base), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory", "m0");
}

// The same for data that is read once (a stream that should not push what others re-read out of the caches).
__device__ __forceinline__ void direct_load_16_offset_streaming(const void* uniform_base, unsigned byte_offset,
                                                                unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :
                 : "v"(byte_offset), "s"(uniform_base), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory", "m0");
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding:
// vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14, expcnt/lgkmcnt unconstrained).
template <int COUNT>
__device__ __forceinline__ void wait_vector_memory() {
    __builtin_amdgcn_s_waitcnt((COUNT & 15) | ((COUNT >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Workgroup barrier without the full memory fence of __syncthreads(): the fence
// would wait for every outstanding vector-memory operation, i.e. for loads that
// are meant to stay in flight across the barrier.  LDS traffic of this wave is
// drained.
__device__ __forceinline__ void workgroup_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Lane id read afresh.  Being volatile, nothing computed from it is hoisted out
// of a loop: per-lane addresses are recomputed where they are used (a handful
// of integer ops) instead of being carried in registers.
__device__ __forceinline__ int fresh_lane_id() {
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

// XCD-aware work-item order.  Workgroups are handed to the 8 XCDs round-robin
// by linear id; every XCD has a private L2.  Items are grouped so that the
// `inner` items that share operands (the query blocks of one head) run on one
// XCD, and `outer` groups (heads) are dealt across XCDs.  Inside an XCD the
// heads are taken two at a time and their items interleaved in inner order:
// with items sorted from heavy to light (a causal triangle) the compute units
// that got the light items of one pair pick up the heavy items of the next, so
// the units finish together, while only two heads' operands are live in the L2.
// Returns (outer index, inner index) for a linear workgroup id; falls back to
// one head at a time when `outer` is a multiple of 8 but not of 16, and to the
// plain order otherwise.
__device__ __forceinline__ void xcd_order(int linear, int outer, int inner, int& outer_index, int& inner_index) {
    constexpr int XCDS = 8;
    if (outer % (2 * XCDS) == 0) {
        const int xcd = linear % XCDS;
        const int slot = linear / XCDS;
        const int pair = slot / (2 * inner);
        const int rest = slot % (2 * inner);
        outer_index = xcd + XCDS * (2 * pair + rest % 2);
        inner_index = rest / 2;
    } else if (outer % XCDS == 0) {
        const int xcd = linear % XCDS;
        const int slot = linear / XCDS;
        outer_index = xcd + XCDS * (slot / inner);
        inner_index = slot % inner;
    } else {
        outer_index = linear / inner;
        inner_index = linear % inner;
    }
}

// f(std::integral_constant<int, BEGIN>) ... f(std::integral_constant<int, END - 1>), in order:
// a loop whose index is a compile-time constant inside the body.
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void unrolled(F&& f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        unrolled<BEGIN + 1, END>(f);
    }
}

#endif  // device helpers

}  // namespace dscuda
