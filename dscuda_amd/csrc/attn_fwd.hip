// Causal attention forward for gfx950: S^T = K Q^T and O^T = V^T P^T on bf16
// MFMA 32x32x16 tiles, online softmax in fp32, natural-log LSE.
//
// One kernel template serves the flash-attention forward (D = 64 / 128, GQA)
// and the per-head MLA prefill forward (d_qk = 128 nope + 64 rope = 192,
// d_v = 128).  It takes the place of the reference's
// flash_attention_forward_tensor_core_kernel
// (kernels/attention/flash_attention/sm89_forward.cu:99-205); the tiling is
// chosen for 64-lane waves and the 160 KB LDS, not taken from there.
//
// Work decomposition
//   workgroup = NWAVES waves, each wave owns 32 query rows for the whole key
//   loop (BM = 32*NWAVES queries per workgroup).  Keys are walked in tiles of
//   BN = 64 from key 0 up to the diagonal.
//
// Transposed formulation
//   Scores are produced as S^T (keys x queries): A = K tile (LDS), B = Q
//   (registers, loaded once).  In the MFMA C layout a lane then holds one
//   query column (lane % 32) and 32 of the tile's 64 keys, so the softmax
//   statistics are per-lane scalars and the only cross-lane step is one
//   exchange with the lane 32 away.  The same registers, rounded to bf16, are
//   directly the B operand of O^T += V^T P^T (k index = key), so P never
//   moves between lanes or through LDS.
//
// LDS layout (per stage, two stages)
//   K  : [64 keys][d_qk] bf16, row pitch 2*d_qk + 16 bytes.  A fragment read
//        is 16 lanes x 16 B down a column of rows; the odd multiple of 16 B in
//        the pitch spreads those over all 64 banks.
//   V^T: [d_v][64 keys] bf16, 128-byte rows, 16-byte chunk index XORed with
//        (row >> 1) & 7.  V arrives row-major (d_v contiguous) but MFMA wants
//        the contraction index (key) contiguous per lane, so each thread
//        transposes a 4 keys x 4 d_v block in registers on the way in.  Inside
//        each group of 16 keys the two middle groups of four are swapped so
//        that the eight keys a lane needs (the C-layout row set
//        {4g..4g+3, 8+4g..8+4g+3}) are one aligned 16-byte read.
//
// Global -> LDS goes through registers: the next tile's loads are issued
// before the current tile's math and written to the other stage after it,
// one workgroup barrier per tile.
#include "attn_kernels.h"
#include "hip_common.h"

#include <cmath>
#include <stdexcept>
#include <string>

namespace dscuda {
namespace {

template <int DQK, int DV, int NWAVES>
struct FwdConfig {
    static constexpr int BN = 64;
    static constexpr int BM = 32 * NWAVES;
    static constexpr int THREADS = 64 * NWAVES;
    static constexpr int K_PITCH = DQK * 2 + 16;           // bytes
    static constexpr int K_BYTES = BN * K_PITCH;
    static constexpr int VT_PITCH = BN * 2;                 // bytes, swizzled
    static constexpr int VT_BYTES = DV * VT_PITCH;
    static constexpr int STAGE_BYTES = K_BYTES + VT_BYTES;
    static constexpr int K_CHUNKS = BN * (DQK / 8);         // 16-byte chunks per K tile
    static constexpr int K_PER_THREAD = K_CHUNKS / THREADS;
    static constexpr int V_UNITS = (BN / 4) * (DV / 4);     // 4 keys x 4 d_v blocks per V tile
    static constexpr int V_PER_THREAD = V_UNITS / THREADS;
    static constexpr int O_PITCH = DV * 2 + 16;             // epilogue staging, bytes
    static constexpr int O_BYTES = BM * O_PITCH;
    static constexpr int LDS_BYTES = (2 * STAGE_BYTES > O_BYTES) ? 2 * STAGE_BYTES : O_BYTES;
    static_assert(K_CHUNKS % THREADS == 0, "K tile must divide evenly over the workgroup");
    static_assert(V_UNITS % THREADS == 0, "V tile must divide evenly over the workgroup");
    static_assert(DQK % 16 == 0 && DV % 32 == 0, "head sizes must fit the MFMA tile");
};

template <int DQK, int DV, int NWAVES>
__global__ __launch_bounds__(64 * NWAVES) void attention_forward_kernel(
    bf16_t* __restrict__ output, float* __restrict__ logsumexp,
    const bf16_t* __restrict__ query, const bf16_t* __restrict__ key, const bf16_t* __restrict__ value,
    int sequence_length, int query_heads, int key_value_heads, int query_blocks, float scale) {
    using C = FwdConfig<DQK, DV, NWAVES>;
    constexpr int BN = C::BN;
    constexpr int KSTEPS = DQK / 16;
    constexpr int DBLOCKS = DV / 32;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;

    // (batch, head) groups are dealt across XCDs; inside a group the heaviest
    // (last) query blocks are issued first.
    int bh, qb_rank;
    xcd_order(blockIdx.x, gridDim.x / query_blocks, query_blocks, bh, qb_rank);
    const int qb = query_blocks - 1 - qb_rank;
    const int b = bh / query_heads;
    const int h = bh % query_heads;
    const int hk = h / (query_heads / key_value_heads);
    const int S = sequence_length;

    const int q0 = qb * C::BM;
    const int wave_q0 = q0 + 32 * wave;
    const int q_row = wave_q0 + lq;

    const size_t q_stride = (size_t)query_heads * DQK;
    const size_t k_stride = (size_t)key_value_heads * DQK;
    const size_t v_stride = (size_t)key_value_heads * DV;
    const bf16_t* q_base = query + ((size_t)b * S * query_heads + h) * DQK;
    const bf16_t* k_base = key + ((size_t)b * S * key_value_heads + hk) * DQK;
    const bf16_t* v_base = value + ((size_t)b * S * key_value_heads + hk) * DV;

    // ---- Q fragments (B operand: column = query lq, k = 16*ks + 8*g + j)
    bf16x8 qf[KSTEPS];
    {
        const bool valid = q_row < S;
        const bf16_t* row = q_base + (size_t)(valid ? q_row : 0) * q_stride + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            u32x4 bits = {0, 0, 0, 0};
            if (valid) {
                bits = *reinterpret_cast<const u32x4*>(row + 16 * ks);
            }
            qf[ks] = __builtin_bit_cast(bf16x8, bits);
        }
    }

    const int last_key = min(S, q0 + C::BM) - 1;
    const int tiles = last_key / BN + 1;

    u32x4 k_stage[C::K_PER_THREAD];
    u32x2 v_stage[C::V_PER_THREAD][4];

    auto load_tile = [&](int tile) {
        const int key0 = tile * BN;
#pragma unroll
        for (int i = 0; i < C::K_PER_THREAD; ++i) {
            const int id = tid + C::THREADS * i;
            const int row = id / (DQK / 8);
            const int col = id % (DQK / 8);
            const int k = key0 + row;
            u32x4 bits = {0, 0, 0, 0};
            if (k < S) {
                bits = *reinterpret_cast<const u32x4*>(k_base + (size_t)k * k_stride + 8 * col);
            }
            k_stage[i] = bits;
        }
#pragma unroll
        for (int i = 0; i < C::V_PER_THREAD; ++i) {
            const int unit = tid + C::THREADS * i;
            const int c4 = unit % (DV / 4);
            const int kg = unit / (DV / 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = key0 + 4 * kg + j;
                u32x2 bits = {0, 0};
                if (k < S) {
                    bits = *reinterpret_cast<const u32x2*>(v_base + (size_t)k * v_stride + 4 * c4);
                }
                v_stage[i][j] = bits;
            }
        }
    };

    auto store_tile = [&](int stage) {
        unsigned char* k_lds = lds + stage * C::STAGE_BYTES;
        unsigned char* vt_lds = k_lds + C::K_BYTES;
#pragma unroll
        for (int i = 0; i < C::K_PER_THREAD; ++i) {
            const int id = tid + C::THREADS * i;
            const int row = id / (DQK / 8);
            const int col = id % (DQK / 8);
            *reinterpret_cast<u32x4*>(k_lds + row * C::K_PITCH + 16 * col) = k_stage[i];
        }
#pragma unroll
        for (int i = 0; i < C::V_PER_THREAD; ++i) {
            const int unit = tid + C::THREADS * i;
            const int c4 = unit % (DV / 4);
            const int kg = unit / (DV / 4);
            // keys 4*kg .. 4*kg+3 = 16*n + 8*a + 4*g' + (0..3)  ->  position 16*n + 8*g' + 4*a
            const int n = kg / 4;
            const int a = (kg % 4) / 2;
            const int gp = kg % 2;
            const int chunk = 2 * n + gp;
            const u32x2 r0 = v_stage[i][0], r1 = v_stage[i][1], r2 = v_stage[i][2], r3 = v_stage[i][3];
            u32x2 t[4];
            t[0] = u32x2{(r0.x & 0xffffu) | (r1.x << 16), (r2.x & 0xffffu) | (r3.x << 16)};
            t[1] = u32x2{(r0.x >> 16) | (r1.x & 0xffff0000u), (r2.x >> 16) | (r3.x & 0xffff0000u)};
            t[2] = u32x2{(r0.y & 0xffffu) | (r1.y << 16), (r2.y & 0xffffu) | (r3.y << 16)};
            t[3] = u32x2{(r0.y >> 16) | (r1.y & 0xffff0000u), (r2.y >> 16) | (r3.y & 0xffff0000u)};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int dv = 4 * c4 + e;
                const int swz = chunk ^ ((dv >> 1) & 7);
                *reinterpret_cast<u32x2*>(vt_lds + dv * C::VT_PITCH + 16 * swz + 8 * a) = t[e];
            }
        }
    };

    f32x16 o_acc[DBLOCKS];
#pragma unroll
    for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[d][i] = 0.f;
    }
    float row_max = -INFINITY;  // reference point of the exponent, raw score units
    float row_sum = 0.f;        // this lane's share (its 32 keys per tile) of the normaliser
    const float c = scale * LOG2E;

    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int tile = 0; tile < tiles; ++tile) {
        const int stage = tile & 1;
        const bool more = tile + 1 < tiles;
        if (more) {
            load_tile(tile + 1);
        }
        const int key0 = tile * BN;
        if (key0 <= wave_q0 + 31) {  // otherwise every key of the tile is in this wave's future
            const unsigned char* k_lds = lds + stage * C::STAGE_BYTES;
            const unsigned char* vt_lds = k_lds + C::K_BYTES;

            f32x16 s_acc[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s_acc[mb][i] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(
                        k_lds + (32 * mb + lq) * C::K_PITCH + 32 * ks + 16 * g);
                    s_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s_acc[mb], 0, 0, 0);
                }
            }

            if (key0 + BN - 1 > wave_q0) {  // tile crosses this wave's diagonal
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int k = key0 + 32 * mb + 8 * (i / 4) + 4 * g + (i % 4);
                        if (k > q_row) s_acc[mb][i] = -INFINITY;
                    }
                }
            }

            float tile_max = s_acc[0][0];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
                for (int i = 0; i < 16; ++i) tile_max = fmaxf(tile_max, s_acc[mb][i]);
            }
            tile_max = half_wave_max(tile_max);

            // The reference point only moves when some row's maximum grew by
            // more than 2^8 in the exponent; until then probabilities may
            // exceed one, which fp32 sums and bf16 operands hold without loss.
            const float new_max = fmaxf(row_max, tile_max);
            const bool grew = (new_max - row_max) * c > 8.0f;
            if (__any(grew)) {
                const float alpha = __builtin_amdgcn_exp2f((row_max - new_max) * c);
                row_max = new_max;
                row_sum *= alpha;
#pragma unroll
                for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) o_acc[d][i] *= alpha;
                }
            }

            const float offset = row_max * c;
            bf16x8 pf[4];
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                u32x4 packed;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int i = 8 * (n % 2) + 2 * j;
                    const float p0 = __builtin_amdgcn_exp2f(fmaf(s_acc[n / 2][i], c, -offset));
                    const float p1 = __builtin_amdgcn_exp2f(fmaf(s_acc[n / 2][i + 1], c, -offset));
                    row_sum += p0 + p1;
                    packed[j] = pack_bf16(p0, p1);
                }
                pf[n] = __builtin_bit_cast(bf16x8, packed);
            }

#pragma unroll
            for (int n = 0; n < 4; ++n) {
#pragma unroll
                for (int d = 0; d < DBLOCKS; ++d) {
                    const int dv = 32 * d + lq;
                    const int swz = (2 * n + g) ^ ((dv >> 1) & 7);
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(vt_lds + dv * C::VT_PITCH + 16 * swz);
                    o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[n], o_acc[d], 0, 0, 0);
                }
            }
        }
        if (more) {
            store_tile(stage ^ 1);
        }
        __syncthreads();
    }

    // ---- epilogue: normalise, stage O through LDS for 16-byte row stores
    const float total = half_wave_sum(row_sum);
    const float inverse = 1.0f / total;
    if (g == 0 && q_row < S) {
        logsumexp[((size_t)b * query_heads + h) * S + q_row] = row_max * scale + __logf(total);
    }
    unsigned char* o_lds = lds + (32 * wave) * C::O_PITCH;
#pragma unroll
    for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            u32x2 packed;
            packed.x = pack_bf16(o_acc[d][4 * i4 + 0] * inverse, o_acc[d][4 * i4 + 1] * inverse);
            packed.y = pack_bf16(o_acc[d][4 * i4 + 2] * inverse, o_acc[d][4 * i4 + 3] * inverse);
            const int dv = 32 * d + 8 * i4 + 4 * g;
            *reinterpret_cast<u32x2*>(o_lds + lq * C::O_PITCH + 2 * dv) = packed;
        }
    }
    __syncthreads();
    constexpr int ROW_CHUNKS = DV / 8;          // 16-byte chunks per output row
    constexpr int ROWS_PER_PASS = 64 / ROW_CHUNKS;
    const size_t o_stride = (size_t)query_heads * DV;
    bf16_t* o_base = output + ((size_t)b * S * query_heads + h) * DV;
#pragma unroll
    for (int pass = 0; pass < 32 / ROWS_PER_PASS; ++pass) {
        const int row = pass * ROWS_PER_PASS + lane / ROW_CHUNKS;
        const int chunk = lane % ROW_CHUNKS;
        const int q = wave_q0 + row;
        if (q < S) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(o_lds + row * C::O_PITCH + 16 * chunk);
            *reinterpret_cast<u32x4*>(o_base + (size_t)q * o_stride + 8 * chunk) = bits;
        }
    }
}

template <int DQK, int DV, int NWAVES>
void launch_forward(bf16_t* output, float* logsumexp, const bf16_t* query, const bf16_t* key, const bf16_t* value,
                    int batch_size, int sequence_length, int query_heads, int key_value_heads, float scale,
                    hipStream_t stream) {
    using C = FwdConfig<DQK, DV, NWAVES>;
    const int query_blocks = (sequence_length + C::BM - 1) / C::BM;
    const long long groups = (long long)batch_size * query_heads;
    const long long grid = groups * query_blocks;
    if (grid > 0x7fffffffLL) {
        throw std::invalid_argument("attention forward: batch*heads*query_blocks exceeds the grid limit");
    }
    auto kernel = attention_forward_kernel<DQK, DV, NWAVES>;
    if (C::LDS_BYTES > 64 * 1024) {
        static thread_local bool raised = false;  // attribute is per function, setting it is idempotent
        if (!raised) {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES));
            raised = true;
        }
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(C::THREADS), C::LDS_BYTES, stream, output, logsumexp, query,
                       key, value, sequence_length, query_heads, key_value_heads, query_blocks, scale);
    HIP_CHECK(hipGetLastError());
}

}  // namespace

void attention_forward_dispatch(bf16_t* output, float* logsumexp, const bf16_t* query, const bf16_t* key,
                                const bf16_t* value, int batch_size, int sequence_length, int query_heads,
                                int key_value_heads, int qk_head_size, int v_head_size, float scale,
                                hipStream_t stream) {
    // Few, large workgroups (256 queries) when there is enough work to fill the
    // chip; 128-query workgroups otherwise so that short problems still spread.
    const long long rows = (long long)batch_size * query_heads * sequence_length;
    const bool large = rows >= 256LL * 256 * 2;
#define DSCUDA_FWD_CASE(DQK, DV)                                                                                  \
    if (qk_head_size == DQK && v_head_size == DV) {                                                               \
        if constexpr (DV >= 128) {                                                                                \
            if (large) {                                                                                          \
                launch_forward<DQK, DV, 8>(output, logsumexp, query, key, value, batch_size, sequence_length,     \
                                           query_heads, key_value_heads, scale, stream);                          \
                return;                                                                                           \
            }                                                                                                     \
        }                                                                                                         \
        launch_forward<DQK, DV, 4>(output, logsumexp, query, key, value, batch_size, sequence_length,             \
                                   query_heads, key_value_heads, scale, stream);                                  \
        return;                                                                                                   \
    }
    DSCUDA_FWD_CASE(192, 128)
    DSCUDA_FWD_CASE(128, 128)
    DSCUDA_FWD_CASE(64, 64)
#undef DSCUDA_FWD_CASE
    throw std::invalid_argument("attention forward: unsupported head sizes (d_qk,d_v) = (" +
                                std::to_string(qk_head_size) + "," + std::to_string(v_head_size) + ")");
}

}  // namespace dscuda
