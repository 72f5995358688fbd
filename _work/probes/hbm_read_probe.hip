// What a kernel that only reads can draw from HBM on this GPU: the yardstick for the decode
// kernel, which is a read stream with matrix work hidden behind it.  Two forms are timed over the
// same buffer:
//
//   registers   every lane fetches 16 bytes per instruction into registers (UNROLL independent
//               fetches in flight per lane) and XORs them together;
//   lds         the decode kernel's own instruction: each wave streams 1 KB per instruction
//               straight into LDS (global_load_lds_dwordx4), 36 KB units through a ring of four
//               slots with one, two or three units in flight per workgroup, one workgroup per
//               compute unit;
//   both        four waves of a workgroup stream into LDS while four others read into registers,
//               each over its own share of the buffer.
//
// Usage: hbm_read_probe [MiB = 1024] [iterations = 20]
// Prints one line per form and launch shape, and "HBM_READ_PROBE best_GBps=..." at the end.
// The register form checks the XOR of everything it read against the closed form of the fill.

#include <cstdint>

#include "profiler_common.h"

#include "hip_common.h"

namespace {

template <int UNROLL>
__global__ __launch_bounds__(256) void read_into_registers(const uint4* data, size_t count, uint4* sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint4 total = {0, 0, 0, 0};
    for (; i + (UNROLL - 1) * stride < count; i += UNROLL * stride) {
        uint4 piece[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) piece[u] = data[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            total.x ^= piece[u].x;
            total.y ^= piece[u].y;
            total.z ^= piece[u].z;
            total.w ^= piece[u].w;
        }
    }
    for (; i < count; i += stride) {
        const uint4 piece = data[i];
        total.x ^= piece.x;
        total.y ^= piece.y;
        total.z ^= piece.z;
        total.w ^= piece.w;
    }
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = total;
}

__global__ __launch_bounds__(256) void fill_words(unsigned* words, size_t count) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) words[i] = (unsigned)i * 2654435761u;
}

constexpr int UNIT_BYTES = 36864;   // 32 cache rows of 1152 bytes
constexpr int SLOTS = 4;
constexpr int WAVE_LOADS = 9;       // 9 KB per wave and unit

// Units blockIdx.x, blockIdx.x + gridDim.x, ... of the buffer; `units` whole units lie inside it.
// IN_FLIGHT units of a workgroup are on their way at a time (the youngest IN_FLIGHT - 1 are not waited for).
template <int IN_FLIGHT>
__global__ __launch_bounds__(256) void read_into_lds(const unsigned char* data, int units, unsigned* sink) {
    extern __shared__ __align__(16) unsigned char lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const unsigned lds_base = dscuda::lds_offset_of(lds);
    int issued = 0;
    for (int unit = blockIdx.x; unit < units; unit += gridDim.x, ++issued) {
        const unsigned char* source = data + (size_t)unit * UNIT_BYTES + wave * (WAVE_LOADS * 1024);
        const unsigned target = lds_base + (issued % SLOTS) * UNIT_BYTES + wave * (WAVE_LOADS * 1024);
#pragma unroll
        for (int i = 0; i < WAVE_LOADS; ++i) dscuda::direct_load_16_offset(source, i * 1024 + lane * 16, target + i * 1024);
        dscuda::wait_vector_memory<(IN_FLIGHT - 1) * WAVE_LOADS>();
    }
    dscuda::wait_vector_memory<0>();
    dscuda::workgroup_barrier();
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = reinterpret_cast<const unsigned*>(lds)[threadIdx.x];
}

// Both forms in one workgroup of eight waves: waves 0-3 stream units [0, units) into LDS (three in flight), waves
// 4-7 read the 16-byte pieces [first_piece, count) into registers.  If the two together draw more than either
// alone, what limits the LDS form is its request path and not the memory.
__global__ __launch_bounds__(512) void read_both(const unsigned char* data, int units, size_t first_piece, size_t count,
                                                 unsigned* sink) {
    extern __shared__ __align__(16) unsigned char lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    unsigned folded = 0;
    if (wave < 4) {
        const unsigned lds_base = dscuda::lds_offset_of(lds);
        int issued = 0;
        for (int unit = blockIdx.x; unit < units; unit += gridDim.x, ++issued) {
            const unsigned char* source = data + (size_t)unit * UNIT_BYTES + wave * (WAVE_LOADS * 1024);
            const unsigned target = lds_base + (issued % SLOTS) * UNIT_BYTES + wave * (WAVE_LOADS * 1024);
#pragma unroll
            for (int i = 0; i < WAVE_LOADS; ++i) dscuda::direct_load_16_offset(source, i * 1024 + lane * 16, target + i * 1024);
            dscuda::wait_vector_memory<2 * WAVE_LOADS>();
        }
        dscuda::wait_vector_memory<0>();
    } else {
        constexpr int UNROLL = 8;
        const uint4* pieces = reinterpret_cast<const uint4*>(data);
        const size_t stride = (size_t)gridDim.x * 256;
        size_t i = first_piece + (size_t)blockIdx.x * 256 + (threadIdx.x - 256);
        uint4 total = {0, 0, 0, 0};
        for (; i + (UNROLL - 1) * stride < count; i += UNROLL * stride) {
            uint4 piece[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) piece[u] = pieces[i + u * stride];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                total.x ^= piece[u].x;
                total.y ^= piece[u].y;
                total.z ^= piece[u].z;
                total.w ^= piece[u].w;
            }
        }
        folded = total.x ^ total.y ^ total.z ^ total.w;
    }
    __syncthreads();
    sink[(size_t)blockIdx.x * 512 + threadIdx.x] = folded ^ reinterpret_cast<const unsigned*>(lds)[threadIdx.x % 256];
}

}  // namespace

int main(int argc, char** argv) {
    try {
        const size_t mib = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 1024;
        const int iterations = argc > 2 ? std::atoi(argv[2]) : 20;
        if (mib < 1 || mib > 65536 || iterations < 1) throw std::invalid_argument("usage: hbm_read_probe [MiB] [iterations]");
        const size_t bytes = mib << 20;
        const size_t count = bytes / sizeof(uint4);
        constexpr int MAX_GRID = 256 * 16;
        profiler::DeviceBuffer<unsigned char> data(bytes);
        profiler::DeviceBuffer<uint4> sink((size_t)MAX_GRID * 256);
        fill_words<<<2048, 256>>>(reinterpret_cast<unsigned*>(data.get()), bytes / 4);
        PROFILER_HIP_CHECK(hipGetLastError());
        unsigned expected = 0;   // XOR of every word of the buffer
        for (size_t i = 0; i < bytes / 4; ++i) expected ^= (unsigned)i * 2654435761u;
        for (const void* kernel : {reinterpret_cast<const void*>(read_into_lds<1>), reinterpret_cast<const void*>(read_into_lds<2>),
                                   reinterpret_cast<const void*>(read_into_lds<3>)}) {
            PROFILER_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SLOTS * UNIT_BYTES));
        }
        hipEvent_t start, stop;
        PROFILER_HIP_CHECK(hipEventCreate(&start));
        PROFILER_HIP_CHECK(hipEventCreate(&stop));
        double best = 0.0;

        auto timed = [&](const char* form, int grid, double moved, auto&& launch) {
            for (int i = 0; i < 3; ++i) launch();
            PROFILER_HIP_CHECK(hipEventRecord(start, nullptr));
            for (int i = 0; i < iterations; ++i) launch();
            PROFILER_HIP_CHECK(hipEventRecord(stop, nullptr));
            PROFILER_HIP_CHECK(hipEventSynchronize(stop));
            PROFILER_HIP_CHECK(hipGetLastError());
            float ms = 0.0f;
            PROFILER_HIP_CHECK(hipEventElapsedTime(&ms, start, stop));
            const double rate = moved / (ms * 1e-3 / iterations) / 1e9;
            std::printf("%-9s workgroups %5d  %9.1f us  %8.1f GB/s\n", form, grid, ms * 1e3 / iterations, rate);
            best = std::max(best, rate);
        };

        for (int per_unit : {2, 4, 8, 16}) {
            const int grid = 256 * per_unit;
            timed("registers", grid, (double)bytes,
                  [&] { read_into_registers<8><<<grid, 256>>>(reinterpret_cast<const uint4*>(data.get()), count, sink.get()); });
            const std::vector<uint4> host = sink.download();
            unsigned folded = 0;
            for (size_t i = 0; i < (size_t)grid * 256; ++i) folded ^= host[i].x ^ host[i].y ^ host[i].z ^ host[i].w;
            if (folded != expected) throw std::runtime_error("register form: XOR of the buffer differs from its closed form");
        }
        const int units = (int)std::min<size_t>(bytes / UNIT_BYTES, 1u << 30);
        unsigned* words = reinterpret_cast<unsigned*>(sink.get());
        timed("lds x1", 256, (double)units * UNIT_BYTES,
              [&] { read_into_lds<1><<<256, 256, SLOTS * UNIT_BYTES>>>(data.get(), units, words); });
        timed("lds x2", 256, (double)units * UNIT_BYTES,
              [&] { read_into_lds<2><<<256, 256, SLOTS * UNIT_BYTES>>>(data.get(), units, words); });
        timed("lds x3", 256, (double)units * UNIT_BYTES,
              [&] { read_into_lds<3><<<256, 256, SLOTS * UNIT_BYTES>>>(data.get(), units, words); });
        PROFILER_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(read_both),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, SLOTS * UNIT_BYTES));
        for (int tenths : {3, 4, 5, 6}) {   // share of the buffer that goes through registers
            const size_t first_piece = (size_t)units * (10 - tenths) / 10 * UNIT_BYTES / sizeof(uint4);
            const int lds_units = (int)(first_piece * sizeof(uint4) / UNIT_BYTES);
            char form[32];
            std::snprintf(form, sizeof form, "both .%d", tenths);
            timed(form, 256, (double)lds_units * UNIT_BYTES + (double)(count - first_piece) * sizeof(uint4),
                  [&] { read_both<<<256, 512, SLOTS * UNIT_BYTES>>>(data.get(), lds_units, first_piece, count, words); });
        }
        std::printf("check passed\nHBM_READ_PROBE bytes=%zu best_GBps=%.1f\n", bytes, best);
        PROFILER_HIP_CHECK(hipEventDestroy(start));
        PROFILER_HIP_CHECK(hipEventDestroy(stop));
        return 0;
    } catch (const std::exception& error) {
        std::fprintf(stderr, "hbm_read_probe: %s\n", error.what());
        return 1;
    }
}
