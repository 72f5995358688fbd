// The two per-head projections either side of absorbed MLA attention, which the reference
// leaves to its caller (reference/python/sources.json:2: "No ... model projections"):
//
//     absorb     q_latent[t, h, c] = sum_d q_nope[t, h, d]  * W_UK[h, d, c]      (d < 128, c < 512)
//     un-absorb  out[t, h, d]      = sum_c o_latent[t, h, c] * W_UV[h, d, c]
//
// with both weights in the layout of the two halves of DeepSeek-V3's wkv_b viewed as
// [heads, 128 + 128, 512] (inference/model.py of deepseek-ai/DeepSeek-V3: the absorbed
// attention path multiplies q_nope by wkv_b[:, :128] before and the latent output by
// wkv_b[:, -128:] after the attention).  BF16 in and out, FP32 accumulation on the
// 32x32x16 MFMA.
//
// A head's weight (128 KB) is staged once per workgroup in LDS, row-major as 32-row tiles;
// a wave then takes 32 tokens at a time, holds their input rows in registers straight from
// memory (lane = token, as the operand whose column is the token) and forms the transposed
// product y^T = W x^T; a lane ends up with one token and groups of four neighbouring output
// columns, which leave through a small LDS stage as whole 128-byte lines.
//   absorb:    W_UK[h] is [d][c]; the contraction index d is the tile row, so the weight
//              operand comes through transposing reads (ds_read_b64_tr_b16), which deliver
//              rows {4g..4g+3, 8+4g..8+4g+3} of a 16-row step: the token operand is brought
//              into the same order by one lane exchange per step.
//   un-absorb: W_UV[h] is [d][c]; the contraction index c is the tile column: plain 16-byte
//              row reads on both sides.
// Either way a token tile costs 128 MFMAs per wave against 8 + 32 KB (absorb) or 32 + 8 KB
// of memory traffic: the kernels are bound by memory.

#include "attn_kernels.h"
#include "hip_common.h"

#include <algorithm>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

namespace dscuda {
namespace {

constexpr int RANK = 512;       // c
constexpr int HEAD = 128;       // d
constexpr int THREADS = 256;
constexpr int TILE = 32;
constexpr int PITCH = 2 * RANK + 16;            // bytes per weight row in LDS: 16 bytes apart modulo 256
constexpr int TILE_BYTES = TILE * PITCH;
constexpr int WEIGHT_BYTES = (HEAD / TILE) * TILE_BYTES;   // 133 120
constexpr int AHEAD = 6;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4* transposing_read_pointer;

template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// W[h] ([128][512], `weight`) -> LDS, 16-byte pieces
// (sixteen loads in flight per thread and round trip: one at a time, the 32 round trips of a thread's share were a
// third of the kernel's time)
__device__ __forceinline__ void stage_weight(unsigned char* lds, const bf16_t* weight, int tid) {
    constexpr int PIECES = HEAD * RANK / 8;
    constexpr int PER_THREAD = PIECES / THREADS;   // 32
    constexpr int BATCH = 16;
    static_assert(PER_THREAD * THREADS == PIECES && PER_THREAD % BATCH == 0, "the weight must divide evenly");
#pragma unroll
    for (int first = 0; first < PER_THREAD; first += BATCH) {
        u32x4 bits[BATCH];
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            bits[j] = *reinterpret_cast<const u32x4*>(weight + 8 * (tid + (first + j) * THREADS));
        }
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            const int piece = tid + (first + j) * THREADS;
            const int row = piece / (RANK / 8);
            const int chunk = piece % (RANK / 8);
            *reinterpret_cast<u32x4*>(lds + (row / TILE) * TILE_BYTES + (row % TILE) * PITCH + 16 * chunk) = bits[j];
        }
    }
}

// A wave's results leave through LDS, two 32-column blocks (one 128-byte line per token) at a time: a lane holds
// one token and scattered groups of four columns, and stores straight from the accumulators would touch 32
// different rows with 16 bytes each.
constexpr int STAGE_PITCH = 128 + 16;
constexpr int STAGE_BYTES = TILE * STAGE_PITCH;              // per wave
constexpr int LDS_BYTES = WEIGHT_BYTES + 4 * STAGE_BYTES;

// blocks `first`, `first + 1` of the accumulators -> columns 32 * first .. + 63 of the tile's tokens
template <int BLOCKS>
__device__ __forceinline__ void store_block_pair(const f32x16 (&acc)[BLOCKS], int first, unsigned char* stage, bf16_t* y_head,
                                                 long long y_token_stride, long long tile0, long long tokens, int lane) {
    const int lq = lane % 32;
    const int g = lane / 32;
#pragma unroll
    for (int pair = 0; pair < 2; ++pair) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            u32x2 packed;
            packed.x = pack_bf16(acc[first + pair][4 * i4 + 0], acc[first + pair][4 * i4 + 1]);
            packed.y = pack_bf16(acc[first + pair][4 * i4 + 2], acc[first + pair][4 * i4 + 3]);
            *reinterpret_cast<u32x2*>(stage + lq * STAGE_PITCH + 64 * pair + 16 * i4 + 8 * g) = packed;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): this wave's LDS writes have landed
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 8 * r + lane / 8;
        const int chunk = lane % 8;
        const u32x4 bits = *reinterpret_cast<const u32x4*>(stage + row * STAGE_PITCH + 16 * chunk);
        if (tile0 + row < tokens) {
            *reinterpret_cast<u32x4*>(y_head + (tile0 + row) * y_token_stride + 32 * first + 8 * chunk) = bits;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);   // the reads are done before the next pair overwrites the stage
    __builtin_amdgcn_wave_barrier();
}

// The 16 bytes at 16ks + 8g of a token's row for every k-step (zeros for a token past the end).
template <int KSTEPS>
__device__ __forceinline__ void fetch_token_row(u32x4 (&bits)[KSTEPS], const bf16_t* row, bool valid, int g) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        bits[ks] = u32x4{0, 0, 0, 0};
        if (valid) bits[ks] = *reinterpret_cast<const u32x4*>(row + 16 * ks + 8 * g);
    }
}

struct Strides {
    long long x_token, x_head, y_token, y_head, w_head;   // in elements
};

// q_latent = q_nope W_UK
__global__ __launch_bounds__(THREADS) void mla_absorb_query_kernel(bf16_t* __restrict__ y, const bf16_t* __restrict__ x,
                                                                   const bf16_t* __restrict__ weight, long long tokens,
                                                                   long long tokens_per_workgroup, Strides strides) {
    constexpr int KSTEPS = HEAD / 16;      // 8
    constexpr int BLOCKS = RANK / 32;      // 16 output column blocks
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int head = blockIdx.y;
    stage_weight(lds, weight + head * strides.w_head, tid);
    unsigned char* stage = lds + WEIGHT_BYTES + wave * STAGE_BYTES;
    __syncthreads();

    // transposing reads: in a block of 16 lanes, lane s points at row 4*g + s/4 (+8), columns 4*(s%4)..+3 of
    // the block's 16 columns
    const int s = lane % 16;
    const int half = (lane / 16) % 2;
    const int lane_offset = (4 * g + s / 4) * PITCH + 32 * half + 8 * (s % 4);
    auto weight_fragment = [&](auto tag) {
        constexpr int I = decltype(tag)::value;   // k-step I / BLOCKS, column block I % BLOCKS
        constexpr int KS = I / BLOCKS;
        constexpr int BLOCK = I % BLOCKS;
        const unsigned char* at = lds + (KS / 2) * TILE_BYTES + (KS % 2) * 16 * PITCH + lane_offset + 64 * BLOCK;
        const s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)at);
        const s16x4 high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(at + 8 * PITCH));
        return __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    // a wave's tiles: tile0, tile0 + 128, ... below `end`; the rows of the next tile are fetched while this one is multiplied
    const long long first = (long long)blockIdx.x * tokens_per_workgroup;
    const long long end = min(first + tokens_per_workgroup, tokens);
    const bf16_t* x_head = x + head * strides.x_head;
    auto row_of = [&](long long tile0) { return x_head + min(tile0 + lq, tokens - 1) * strides.x_token; };
    u32x4 next_bits[KSTEPS];
    fetch_token_row(next_bits, row_of(first + TILE * wave), first + TILE * wave + lq < tokens, g);
    for (long long tile0 = first + TILE * wave; tile0 < end; tile0 += TILE * 4) {
        // The token operand has to hold columns {16ks + 4g .. +3, 16ks + 8 + 4g .. +3}, the order of the transposing
        // reads.  Each lane loads the 16 bytes at 16ks + 8g; exchanging the second half of the g = 0 lane's with the
        // first half of the g = 1 lane's (v_permlane32_swap on the two dwords of each half) gives that order.
        bf16x8 xf[KSTEPS];
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const auto first_pair = __builtin_amdgcn_permlane32_swap(next_bits[ks][0], next_bits[ks][2], false, false);
            const auto second_pair = __builtin_amdgcn_permlane32_swap(next_bits[ks][1], next_bits[ks][3], false, false);
            xf[ks] = __builtin_bit_cast(bf16x8, u32x4{first_pair[0], second_pair[0], first_pair[1], second_pair[1]});
        }
        if (tile0 + TILE * 4 < end) fetch_token_row(next_bits, row_of(tile0 + TILE * 4), tile0 + TILE * 4 + lq < tokens, g);
        f32x16 acc[BLOCKS];
#pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;
        }
        bf16x8 ring[AHEAD];
        static_for<0, AHEAD>([&](auto tag) { ring[decltype(tag)::value] = weight_fragment(tag); });
        static_for<0, KSTEPS * BLOCKS>([&](auto tag) {
            constexpr int I = decltype(tag)::value;
            acc[I % BLOCKS] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[I % AHEAD], xf[I / BLOCKS], acc[I % BLOCKS], 0, 0, 0);
            if constexpr (I + AHEAD < KSTEPS * BLOCKS) {
                ring[I % AHEAD] = weight_fragment(std::integral_constant<int, I + AHEAD>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        // lane holds token lq and columns 32*b + 8*(i/4) + 4*g + i%4
#pragma unroll
        for (int b = 0; b < BLOCKS; b += 2) {
            store_block_pair(acc, b, stage, y + head * strides.y_head, strides.y_token, tile0, tokens, lane);
        }
    }
}

// out = o_latent W_UV^T
__global__ __launch_bounds__(THREADS) void mla_unabsorb_output_kernel(bf16_t* __restrict__ y,
                                                                      const bf16_t* __restrict__ x,
                                                                      const bf16_t* __restrict__ weight,
                                                                      long long tokens, long long tokens_per_workgroup,
                                                                      Strides strides) {
    constexpr int KSTEPS = RANK / 16;      // 32
    constexpr int BLOCKS = HEAD / 32;      // 4 output column blocks = the weight's four row tiles
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int head = blockIdx.y;
    stage_weight(lds, weight + head * strides.w_head, tid);
    unsigned char* stage = lds + WEIGHT_BYTES + wave * STAGE_BYTES;
    __syncthreads();

    auto weight_fragment = [&](auto tag) {
        constexpr int I = decltype(tag)::value;   // k-step I / BLOCKS, output block (weight row tile) I % BLOCKS
        constexpr int KS = I / BLOCKS;
        constexpr int BLOCK = I % BLOCKS;
        return *reinterpret_cast<const bf16x8*>(lds + BLOCK * TILE_BYTES + lq * PITCH + 32 * KS + 16 * g);
    };

    const long long first = (long long)blockIdx.x * tokens_per_workgroup;
    const long long end = min(first + tokens_per_workgroup, tokens);
    const bf16_t* x_head = x + head * strides.x_head;
    auto row_of = [&](long long tile0) { return x_head + min(tile0 + lq, tokens - 1) * strides.x_token; };
    u32x4 next_bits[KSTEPS];
    fetch_token_row(next_bits, row_of(first + TILE * wave), first + TILE * wave + lq < tokens, g);
    for (long long tile0 = first + TILE * wave; tile0 < end; tile0 += TILE * 4) {
        bf16x8 xf[KSTEPS];
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) xf[ks] = __builtin_bit_cast(bf16x8, next_bits[ks]);
        if (tile0 + TILE * 4 < end) fetch_token_row(next_bits, row_of(tile0 + TILE * 4), tile0 + TILE * 4 + lq < tokens, g);
        f32x16 acc[BLOCKS];
#pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;
        }
        bf16x8 ring[AHEAD];
        static_for<0, AHEAD>([&](auto tag) { ring[decltype(tag)::value] = weight_fragment(tag); });
        static_for<0, KSTEPS * BLOCKS>([&](auto tag) {
            constexpr int I = decltype(tag)::value;
            acc[I % BLOCKS] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[I % AHEAD], xf[I / BLOCKS], acc[I % BLOCKS], 0, 0, 0);
            if constexpr (I + AHEAD < KSTEPS * BLOCKS) {
                ring[I % AHEAD] = weight_fragment(std::integral_constant<int, I + AHEAD>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        // lane holds token lq and columns 32*b + 8*(i/4) + 4*g + i%4
#pragma unroll
        for (int b = 0; b < BLOCKS; b += 2) {
            store_block_pair(acc, b, stage, y + head * strides.y_head, strides.y_token, tile0, tokens, lane);
        }
    }
}

void check(bool condition, const char* message) {
    if (!condition) throw std::invalid_argument(message);
}

int compute_units() {
    return hip_common::compute_units_of_current_device();
}

// The tokens of a head are cut into chunks, one workgroup each (multiples of the 128 tokens four waves take); every
// workgroup stages the head's weight first, which costs it about as long as 128 tokens.  The number of chunks is
// the one with the shortest schedule: rounds of workgroups over the compute units times the cost of a workgroup
// (4096 tokens x 128 heads on 256 compute units: two chunks, one round, 138 / 171 us against 145 / 178 us with four).
template <typename Kernel>
void launch(Kernel kernel, bf16_t* y, const bf16_t* x, const bf16_t* weight, long long tokens, int heads,
            const Strides& strides, hipStream_t stream) {
    check(heads <= 65535, "MLA projection: more heads than the grid allows");
    constexpr long long STAGING_TOKENS = 4 * TILE;
    const long long units = std::max(1, compute_units());
    const long long most = (tokens + 4 * TILE - 1) / (4 * TILE);
    const long long limit = std::min(most, std::max(1LL, (4 * units + heads - 1) / heads));
    long long chunks = 1, best = -1;
    for (long long candidate = 1; candidate <= limit; ++candidate) {
        const long long per_chunk = ((tokens + candidate - 1) / candidate + 4 * TILE - 1) / (4 * TILE) * (4 * TILE);
        const long long workgroups = heads * ((tokens + per_chunk - 1) / per_chunk);
        const long long cost = (workgroups + units - 1) / units * (STAGING_TOKENS + per_chunk);
        if (best < 0 || cost < best) {
            best = cost;
            chunks = candidate;
        }
    }
    long long per_workgroup = (tokens + chunks - 1) / chunks;
    per_workgroup = (per_workgroup + 4 * TILE - 1) / (4 * TILE) * (4 * TILE);
    const long long grid = (tokens + per_workgroup - 1) / per_workgroup;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid, (unsigned)heads), dim3(THREADS), LDS_BYTES, stream, y, x, weight,
                       tokens, per_workgroup, strides);
    HIP_CHECK(hipGetLastError());
}

void validate(const void* y, const void* x, const void* weight, long long tokens, int heads, const Strides& s,
              int x_width, int y_width) {
    check(tokens > 0 && heads > 0, "MLA projection: tokens and heads must be positive");
    check(y != nullptr && x != nullptr && weight != nullptr, "MLA projection: null tensor");
    check(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(y) % 16 == 0,
          "MLA projection: tensors must be aligned to 16 bytes");
    check(s.x_token % 8 == 0 && s.x_head % 8 == 0 && s.w_head % 8 == 0 && s.y_token % 8 == 0 && s.y_head % 8 == 0,
          "MLA projection: strides must be multiples of 8 elements (rows aligned to 16 bytes)");
    check(s.x_head >= x_width && s.y_head >= y_width && s.x_token >= s.x_head * (heads - 1) + x_width &&
              s.y_token >= s.y_head * (heads - 1) + y_width && s.w_head >= (long long)HEAD * RANK,
          "MLA projection: strides smaller than the rows they separate");
}

}  // namespace

void mla_absorb_query_dispatch(bf16_t* query_latent, const bf16_t* query_nope, const bf16_t* weight, long long tokens,
                               int heads, long long query_nope_token_stride, long long query_nope_head_stride,
                               long long query_latent_token_stride, long long query_latent_head_stride,
                               long long weight_head_stride, hipStream_t stream) {
    const Strides strides = {query_nope_token_stride, query_nope_head_stride, query_latent_token_stride,
                             query_latent_head_stride, weight_head_stride};
    validate(query_latent, query_nope, weight, tokens, heads, strides, HEAD, RANK);
    static hip_common::OncePerDevice prepared;
    prepared.run([] {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(mla_absorb_query_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    });
    launch(mla_absorb_query_kernel, query_latent, query_nope, weight, tokens, heads, strides, stream);
}

void mla_unabsorb_output_dispatch(bf16_t* output, const bf16_t* output_latent, const bf16_t* weight, long long tokens,
                                  int heads, long long output_latent_token_stride, long long output_latent_head_stride,
                                  long long output_token_stride, long long output_head_stride,
                                  long long weight_head_stride, hipStream_t stream) {
    const Strides strides = {output_latent_token_stride, output_latent_head_stride, output_token_stride,
                             output_head_stride, weight_head_stride};
    validate(output, output_latent, weight, tokens, heads, strides, RANK, HEAD);
    static hip_common::OncePerDevice prepared;
    prepared.run([] {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(mla_unabsorb_output_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    });
    launch(mla_unabsorb_output_kernel, output, output_latent, weight, tokens, heads, strides, stream);
}

}  // namespace dscuda
