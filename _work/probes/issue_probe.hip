// What one wave per SIMD can overlap with its own matrix instructions.  The decode kernel runs
// that way (each wave owns all 512 registers of its SIMD lane), so whatever a wave issues between
// two MFMAs either hides behind the MFMA in flight or adds to it; this program measures which.
//
// One workgroup of four waves per compute unit runs a register-only loop.  Per iteration:
//
//   mfma        4 independent v_mfma_f32_32x32x16_bf16 (8 passes each)
//   chain       4 MFMAs accumulating into the same registers
//   valu        24 independent v_fma_f32
//   mfma+valu   the 4 MFMAs, 6 of the FMAs after each
//   lds         8 ds_read_b128 and one wait for them
//   mfma+lds    the 4 MFMAs, 2 of the reads after each, one wait at the end
//   salu        24 s_add_u32
//   mfma+salu   the 4 MFMAs, 6 of the adds after each
//
// and the program prints the time per iteration of each form in nanoseconds and as a multiple of
// `mfma`.  If `mfma+x` costs about as much as `mfma`, x hides; if it costs `mfma` + `x`, it does not.
//
// Usage: issue_probe [iterations = 20000]

#include <cstdint>

#include "profiler_common.h"

#include "hip_common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

enum Form { MFMA, CHAIN, VALU, MFMA_VALU, LDS, MFMA_LDS, SALU, MFMA_SALU, FORMS };
const char* const NAMES[FORMS] = {"mfma", "chain", "valu", "mfma+valu", "lds", "mfma+lds", "salu", "mfma+salu"};

// operands: 0-3 accumulators, 4-9 FMA registers, 10-11 read targets, 12 scalar counter; 13 A, 14 B, 15 FMA factor, 16 LDS address
#define PROBE_MFMA(ACC) "v_mfma_f32_32x32x16_bf16 %" #ACC ", %13, %14, %" #ACC "\n\t"
#define PROBE_FMA6 \
    "v_fma_f32 %4, %4, %15, %4\n\tv_fma_f32 %5, %5, %15, %5\n\tv_fma_f32 %6, %6, %15, %6\n\t" \
    "v_fma_f32 %7, %7, %15, %7\n\tv_fma_f32 %8, %8, %15, %8\n\tv_fma_f32 %9, %9, %15, %9\n\t"
#define PROBE_READ2 "ds_read_b128 %10, %16\n\tds_read_b128 %11, %16 offset:4096\n\t"
#define PROBE_SADD6 \
    "s_add_u32 %12, %12, 1\n\ts_add_u32 %12, %12, 1\n\ts_add_u32 %12, %12, 1\n\t" \
    "s_add_u32 %12, %12, 1\n\ts_add_u32 %12, %12, 1\n\ts_add_u32 %12, %12, 1\n\t"

template <int FORM>
__global__ __launch_bounds__(256) void probe_kernel(float* out, int iterations) {
    __shared__ __align__(16) unsigned char lds[8192 + 64 * 16];
    const int lane = threadIdx.x % 64;
    for (int i = threadIdx.x; i < (int)sizeof(lds) / 4; i += 256) reinterpret_cast<float*>(lds)[i] = 1.0f;
    __syncthreads();
    f32x16 acc0 = {}, acc1 = {}, acc2 = {}, acc3 = {};
    bf16x8 a, b;
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)(0.001f * (lane % 7));
        b[i] = (__bf16)(0.002f * (lane % 5));
    }
    float v0 = lane, v1 = lane + 1, v2 = lane + 2, v3 = lane + 3, v4 = lane + 4, v5 = lane + 5;
    const float c = 0.5f;
    u32x4 r0 = {}, r1 = {};
    const unsigned address = dscuda::lds_offset_of(lds) + lane * 16;
    unsigned s = 0;
    for (int it = 0; it < iterations; ++it) {
#define PROBE_OPERANDS \
    : "+v"(acc0), "+v"(acc1), "+v"(acc2), "+v"(acc3), "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(r0), \
      "+v"(r1), "+s"(s) \
    : "v"(a), "v"(b), "v"(c), "v"(address)
        if constexpr (FORM == MFMA) {
            asm volatile(PROBE_MFMA(0) PROBE_MFMA(1) PROBE_MFMA(2) PROBE_MFMA(3) PROBE_OPERANDS);
        } else if constexpr (FORM == CHAIN) {
            asm volatile(PROBE_MFMA(0) PROBE_MFMA(0) PROBE_MFMA(0) PROBE_MFMA(0) PROBE_OPERANDS);
        } else if constexpr (FORM == VALU) {
            asm volatile(PROBE_FMA6 PROBE_FMA6 PROBE_FMA6 PROBE_FMA6 PROBE_OPERANDS);
        } else if constexpr (FORM == MFMA_VALU) {
            asm volatile(PROBE_MFMA(0) PROBE_FMA6 PROBE_MFMA(1) PROBE_FMA6 PROBE_MFMA(2) PROBE_FMA6 PROBE_MFMA(3) PROBE_FMA6
                         PROBE_OPERANDS);
        } else if constexpr (FORM == LDS) {
            asm volatile(PROBE_READ2 PROBE_READ2 PROBE_READ2 PROBE_READ2 "s_waitcnt lgkmcnt(0)\n\t" PROBE_OPERANDS);
        } else if constexpr (FORM == MFMA_LDS) {
            asm volatile(PROBE_MFMA(0) PROBE_READ2 PROBE_MFMA(1) PROBE_READ2 PROBE_MFMA(2) PROBE_READ2 PROBE_MFMA(3) PROBE_READ2
                         "s_waitcnt lgkmcnt(0)\n\t" PROBE_OPERANDS);
        } else if constexpr (FORM == SALU) {
            asm volatile(PROBE_SADD6 PROBE_SADD6 PROBE_SADD6 PROBE_SADD6 PROBE_OPERANDS : "scc");
        } else {
            asm volatile(PROBE_MFMA(0) PROBE_SADD6 PROBE_MFMA(1) PROBE_SADD6 PROBE_MFMA(2) PROBE_SADD6 PROBE_MFMA(3) PROBE_SADD6
                         PROBE_OPERANDS : "scc");
        }
    }
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt lgkmcnt(0)" ::: "memory");   // the last MFMA and read have written their registers
    float total = v0 + v1 + v2 + v3 + v4 + v5 + (float)(r0[0] + r1[0] + s);
    for (int i = 0; i < 16; ++i) total += acc0[i] + acc1[i] + acc2[i] + acc3[i];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = total;
}

template <int FORM>
double time_form(float* out, int iterations, hipEvent_t start, hipEvent_t stop) {
    probe_kernel<FORM><<<256, 256>>>(out, iterations / 10 + 1);
    PROFILER_HIP_CHECK(hipEventRecord(start, nullptr));
    probe_kernel<FORM><<<256, 256>>>(out, iterations);
    PROFILER_HIP_CHECK(hipEventRecord(stop, nullptr));
    PROFILER_HIP_CHECK(hipEventSynchronize(stop));
    PROFILER_HIP_CHECK(hipGetLastError());
    float ms = 0.0f;
    PROFILER_HIP_CHECK(hipEventElapsedTime(&ms, start, stop));
    return ms * 1e6 / iterations;
}

}  // namespace

int main(int argc, char** argv) {
    try {
        const int iterations = argc > 1 ? std::atoi(argv[1]) : 20000;
        if (iterations < 1 || iterations > 10000000) throw std::invalid_argument("usage: issue_probe [iterations]");
        profiler::DeviceBuffer<float> out((size_t)256 * 256);
        hipEvent_t start, stop;
        PROFILER_HIP_CHECK(hipEventCreate(&start));
        PROFILER_HIP_CHECK(hipEventCreate(&stop));
        double ns[FORMS];
        ns[MFMA] = time_form<MFMA>(out.get(), iterations, start, stop);
        ns[CHAIN] = time_form<CHAIN>(out.get(), iterations, start, stop);
        ns[VALU] = time_form<VALU>(out.get(), iterations, start, stop);
        ns[MFMA_VALU] = time_form<MFMA_VALU>(out.get(), iterations, start, stop);
        ns[LDS] = time_form<LDS>(out.get(), iterations, start, stop);
        ns[MFMA_LDS] = time_form<MFMA_LDS>(out.get(), iterations, start, stop);
        ns[SALU] = time_form<SALU>(out.get(), iterations, start, stop);
        ns[MFMA_SALU] = time_form<MFMA_SALU>(out.get(), iterations, start, stop);
        for (int form = 0; form < FORMS; ++form) {
            std::printf("ISSUE_PROBE %-10s %8.2f ns/iteration  %5.2f x mfma\n", NAMES[form], ns[form], ns[form] / ns[MFMA]);
        }
        // 4 MFMAs of 8 passes of 4 cycles: the clock the loop ran at, if MFMAs issue back to back
        std::printf("check passed: mfma form implies %.2f GHz at 128 cycles per iteration\n", 128.0 / ns[MFMA]);
        PROFILER_HIP_CHECK(hipEventDestroy(start));
        PROFILER_HIP_CHECK(hipEventDestroy(stop));
        return 0;
    } catch (const std::exception& error) {
        std::fprintf(stderr, "issue_probe: %s\n", error.what());
        return 1;
    }
}
