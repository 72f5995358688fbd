// Recompute-based causal attention backward for gfx950 (per-head K/V, the
// 128 nope + 64 rope | 128 value MLA prefill geometry and the square flash
// geometries).  The mathematics is the analytic backward the reference states
// in reference/python/mla.py:42-57 -- P = exp(S - LSE), delta = sum(dO * O),
// dS = P (dP - delta) scale -- with per-head K and V; the reference has no
// kernel for this form (its absorbed backward, kernels/attention/mla/sm89.cu:
// 295-411, is one scalar workgroup per gradient row).
//
// Three launches, every gradient row has exactly one writer (no atomics):
//
//   delta      delta[b,h,s] = sum_c dO * O                        (fp32 workspace)
//   dK/dV      a workgroup owns 128 keys (4 waves x 32) of one head, keeps them
//              in registers, and walks the query tiles from the diagonal to the
//              end of the sequence:   S = Q K^T, dP = dO V^T   (q x keys)
//                                     dV += P^T dO,  dK += dS^T Q
//   dQ         a workgroup owns 128 queries (4 waves x 32), keeps Q and dO in
//              registers, and walks the key tiles up to the diagonal, producing
//              scores transposed as the forward does:
//                                     S^T = K Q^T, dP^T = V dO^T  (keys x q)
//                                     dQ^T += K^T dS^T
//
// In both kernels the probabilities leave the MFMA in its C layout and go back
// in as an operand whose contraction index is the C layout's row index, so P
// and dS never cross lanes.  The other operand of those products is needed
// with the tile's row index (query or key) contiguous per lane; the tile is
// therefore stored in LDS twice, row-major and transposed (a 4x4 register
// transpose per thread on the way in, rows regrouped so that the eight indices
// a lane needs are one 16-byte read), exactly the V^T arrangement of the
// forward kernel.  Row-major copies use a pitch of 2*D + 16 bytes, transposed
// copies 128-byte rows with the 16-byte chunk index XORed with (row>>1)&7;
// both make the 16-row column reads conflict free.
#include "attn_kernels.h"
#include "hip_common.h"

#include <stdexcept>
#include <string>

namespace dscuda {
namespace {

constexpr int BWD_THREADS = 256;
constexpr int BWD_TILE = 64;   // rows of the streamed operand per tile

// ---- shared tile plumbing ----------------------------------------------------

// A [64 rows][D] bf16 tile held twice in LDS.
template <int D>
struct DualTile {
    static constexpr int PITCH = 2 * D + 16;               // row-major copy
    static constexpr int NATURAL_BYTES = BWD_TILE * PITCH;
    static constexpr int T_PITCH = 2 * BWD_TILE;            // transposed copy, 128-byte rows
    static constexpr int TRANSPOSED_BYTES = D * T_PITCH;
    static constexpr int BYTES = NATURAL_BYTES + TRANSPOSED_BYTES;
    static constexpr int UNITS = (BWD_TILE / 4) * (D / 4);  // 4 rows x 4 columns per unit
    static constexpr int PER_THREAD = UNITS / BWD_THREADS;
    static_assert(UNITS % BWD_THREADS == 0, "tile must divide evenly over the workgroup");
};

// Loads the 4x4 units of a tile (rows row0.., `rows` valid) owned by this thread.
template <int D>
__device__ __forceinline__ void load_units(u32x2 (&stage)[DualTile<D>::PER_THREAD][4], const bf16_t* base,
                                           size_t row_stride, int row0, int rows, int tid) {
#pragma unroll
    for (int i = 0; i < DualTile<D>::PER_THREAD; ++i) {
        const int unit = tid + BWD_THREADS * i;
        const int c4 = unit % (D / 4);
        const int rg = unit / (D / 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = row0 + 4 * rg + j;
            u32x2 bits = {0, 0};
            if (row < rows) {
                bits = *reinterpret_cast<const u32x2*>(base + (size_t)row * row_stride + 4 * c4);
            }
            stage[i][j] = bits;
        }
    }
}

// Writes the units row-major (if NATURAL) and transposed (if TRANSPOSED).
template <int D, bool NATURAL, bool TRANSPOSED>
__device__ __forceinline__ void store_units(const u32x2 (&stage)[DualTile<D>::PER_THREAD][4], unsigned char* natural,
                                            unsigned char* transposed, int tid) {
    using T = DualTile<D>;
#pragma unroll
    for (int i = 0; i < T::PER_THREAD; ++i) {
        const int unit = tid + BWD_THREADS * i;
        const int c4 = unit % (D / 4);
        const int rg = unit / (D / 4);
        if (NATURAL) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                *reinterpret_cast<u32x2*>(natural + (4 * rg + j) * T::PITCH + 8 * c4) = stage[i][j];
            }
        }
        if (TRANSPOSED) {
            // rows 4*rg .. 4*rg+3 = 16*n + 8*a + 4*g' + (0..3)  ->  position 16*n + 8*g' + 4*a
            const int n = rg / 4;
            const int a = (rg % 4) / 2;
            const int gp = rg % 2;
            const int chunk = 2 * n + gp;
            const u32x2 r0 = stage[i][0], r1 = stage[i][1], r2 = stage[i][2], r3 = stage[i][3];
            u32x2 t[4];
            t[0] = u32x2{(r0.x & 0xffffu) | (r1.x << 16), (r2.x & 0xffffu) | (r3.x << 16)};
            t[1] = u32x2{(r0.x >> 16) | (r1.x & 0xffff0000u), (r2.x >> 16) | (r3.x & 0xffff0000u)};
            t[2] = u32x2{(r0.y & 0xffffu) | (r1.y << 16), (r2.y & 0xffffu) | (r3.y << 16)};
            t[3] = u32x2{(r0.y >> 16) | (r1.y & 0xffff0000u), (r2.y >> 16) | (r3.y & 0xffff0000u)};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int column = 4 * c4 + e;
                const int swz = chunk ^ ((column >> 1) & 7);
                *reinterpret_cast<u32x2*>(transposed + column * T::T_PITCH + 16 * swz + 8 * a) = t[e];
            }
        }
    }
}

// Operand fragment from the row-major copy: row `row`, elements 16*ks + 8*g ..
template <int D>
__device__ __forceinline__ bf16x8 natural_fragment(const unsigned char* natural, int row, int ks, int g) {
    return *reinterpret_cast<const bf16x8*>(natural + row * DualTile<D>::PITCH + 32 * ks + 16 * g);
}

// Operand fragment from the transposed copy: column `column`, the eight tile
// rows {16n + 4g .. +3, 16n + 8 + 4g .. +3}.
template <int D>
__device__ __forceinline__ bf16x8 transposed_fragment(const unsigned char* transposed, int column, int n, int g) {
    const int swz = (2 * n + g) ^ ((column >> 1) & 7);
    return *reinterpret_cast<const bf16x8*>(transposed + column * DualTile<D>::T_PITCH + 16 * swz);
}

// Registers of an operand that stays with the wave: row `row` of a [.][D] matrix.
template <int D>
__device__ __forceinline__ void load_row_fragments(bf16x8 (&fragments)[D / 16], const bf16_t* base, size_t row_stride,
                                                   int row, bool valid, int g) {
    const bf16_t* source = base + (size_t)(valid ? row : 0) * row_stride + 8 * g;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 bits = {0, 0, 0, 0};
        if (valid) {
            bits = *reinterpret_cast<const u32x4*>(source + 16 * ks);
        }
        fragments[ks] = __builtin_bit_cast(bf16x8, bits);
    }
}

__device__ __forceinline__ void clear(f32x16& value) {
#pragma unroll
    for (int i = 0; i < 16; ++i) value[i] = 0.f;
}

// ---- delta -------------------------------------------------------------------

// One 16-lane group per (b, s, h) row: delta = sum_c dO * O, written as [B,H,S].
template <int DV>
__global__ __launch_bounds__(256) void attention_delta_kernel(float* __restrict__ delta,
                                                              const bf16_t* __restrict__ output_gradient,
                                                              const bf16_t* __restrict__ output, int batch_size,
                                                              int sequence_length, int heads) {
    const long long rows = (long long)batch_size * sequence_length * heads;
    const long long row = (long long)blockIdx.x * 16 + threadIdx.x / 16;
    const int part = threadIdx.x % 16;
    float sum = 0.f;
    if (row < rows) {
#pragma unroll
        for (int c = part * 8; c < DV; c += 128) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(output_gradient + row * DV + c);
            const u32x4 b = *reinterpret_cast<const u32x4*>(output + row * DV + c);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sum += bf16_bits_to_float(a[j] & 0xffffu) * bf16_bits_to_float(b[j] & 0xffffu);
                sum += bf16_bits_to_float(a[j] >> 16) * bf16_bits_to_float(b[j] >> 16);
            }
        }
    }
#pragma unroll
    for (int offset = 1; offset < 16; offset <<= 1) sum += __shfl_xor(sum, offset);
    if (row < rows && part == 0) {
        const long long h = row % heads;
        const long long s = (row / heads) % sequence_length;
        const long long b = row / ((long long)heads * sequence_length);
        delta[(b * heads + h) * sequence_length + s] = sum;
    }
}

// ---- dK / dV -----------------------------------------------------------------

template <int DQK, int DV>
struct KeyGradConfig {
    using QT = DualTile<DQK>;
    using OT = DualTile<DV>;
    static constexpr int KEYS = 128;  // per workgroup
    static constexpr int Q_NATURAL = 0;
    static constexpr int Q_TRANSPOSED = Q_NATURAL + QT::NATURAL_BYTES;
    static constexpr int DO_NATURAL = Q_TRANSPOSED + QT::TRANSPOSED_BYTES;
    static constexpr int DO_TRANSPOSED = DO_NATURAL + OT::NATURAL_BYTES;
    static constexpr int STATS = DO_TRANSPOSED + OT::TRANSPOSED_BYTES;   // lse*log2e [64], delta [64]
    static constexpr int LDS_BYTES = STATS + 2 * BWD_TILE * 4;
    static constexpr int DK_PITCH = 2 * DQK;   // epilogue staging
    static constexpr int DV_PITCH = 2 * DV;
    static_assert(4 * 32 * (DK_PITCH + DV_PITCH) <= LDS_BYTES, "epilogue staging must fit");
};

template <int DQK, int DV>
__global__ __launch_bounds__(BWD_THREADS) void attention_key_gradient_kernel(
    bf16_t* __restrict__ key_gradient, bf16_t* __restrict__ value_gradient,
    const bf16_t* __restrict__ output_gradient, const float* __restrict__ logsumexp, const float* __restrict__ delta,
    const bf16_t* __restrict__ query, const bf16_t* __restrict__ key, const bf16_t* __restrict__ value,
    int sequence_length, int heads, int key_blocks, float scale) {
    using C = KeyGradConfig<DQK, DV>;
    using QT = DualTile<DQK>;
    using OT = DualTile<DV>;
    constexpr int QK_STEPS = DQK / 16;
    constexpr int V_STEPS = DV / 16;
    constexpr int DK_BLOCKS = DQK / 32;
    constexpr int DV_BLOCKS = DV / 32;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    unsigned char* q_natural = lds + C::Q_NATURAL;
    unsigned char* q_transposed = lds + C::Q_TRANSPOSED;
    unsigned char* do_natural = lds + C::DO_NATURAL;
    unsigned char* do_transposed = lds + C::DO_TRANSPOSED;
    float* stats = reinterpret_cast<float*>(lds + C::STATS);

    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int S = sequence_length;

    int bh, kb;  // key block 0 sees every query: heaviest first in natural order
    xcd_order(blockIdx.x, gridDim.x / key_blocks, key_blocks, bh, kb);
    const int b = bh / heads;
    const int h = bh % heads;
    const int k0 = kb * C::KEYS;
    const int wave_k0 = k0 + 32 * wave;
    const int key_row = wave_k0 + lq;

    const size_t qk_stride = (size_t)heads * DQK;
    const size_t v_stride = (size_t)heads * DV;
    const bf16_t* q_base = query + ((size_t)b * S * heads + h) * DQK;
    const bf16_t* k_base = key + ((size_t)b * S * heads + h) * DQK;
    const bf16_t* v_base = value + ((size_t)b * S * heads + h) * DV;
    const bf16_t* do_base = output_gradient + ((size_t)b * S * heads + h) * DV;
    const float* lse_base = logsumexp + ((size_t)b * heads + h) * S;
    const float* delta_base = delta + ((size_t)b * heads + h) * S;

    // K and V rows of this wave, as B operands (column = key lq)
    bf16x8 kf[QK_STEPS], vf[V_STEPS];
    load_row_fragments<DQK>(kf, k_base, qk_stride, key_row, key_row < S, g);
    load_row_fragments<DV>(vf, v_base, v_stride, key_row, key_row < S, g);

    f32x16 dk_acc[DK_BLOCKS], dv_acc[DV_BLOCKS];
#pragma unroll
    for (int d = 0; d < DK_BLOCKS; ++d) clear(dk_acc[d]);
#pragma unroll
    for (int d = 0; d < DV_BLOCKS; ++d) clear(dv_acc[d]);

    const float c = scale * LOG2E;
    const int first_tile = k0 / BWD_TILE;
    const int last_tile = (S - 1) / BWD_TILE;

    u32x2 q_stage[QT::PER_THREAD][4], do_stage[OT::PER_THREAD][4];
    float stat_stage = 0.f;
    auto load_tile = [&](int tile) {
        const int row0 = tile * BWD_TILE;
        load_units<DQK>(q_stage, q_base, qk_stride, row0, S, tid);
        load_units<DV>(do_stage, do_base, v_stride, row0, S, tid);
        if (tid < 2 * BWD_TILE) {
            const int row = row0 + tid % BWD_TILE;
            stat_stage = 0.f;
            if (row < S) stat_stage = tid < BWD_TILE ? lse_base[row] * LOG2E : delta_base[row];
        }
    };
    auto store_tile = [&]() {
        store_units<DQK, true, true>(q_stage, q_natural, q_transposed, tid);
        store_units<DV, true, true>(do_stage, do_natural, do_transposed, tid);
        if (tid < 2 * BWD_TILE) stats[tid] = stat_stage;
    };

    load_tile(first_tile);
    for (int tile = first_tile; tile <= last_tile; ++tile) {
        __syncthreads();   // every wave is done with the previous tile
        store_tile();
        __syncthreads();
        if (tile < last_tile) load_tile(tile + 1);
        const int q0 = tile * BWD_TILE;
        // Tiles whose queries all precede this wave's keys (at most one per wave)
        // are not skipped: they contribute exact zeros through the mask, and a
        // branch around the accumulator updates makes the compiler shuttle all
        // 160 accumulators through scratch.

#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            // S and dP for 32 queries x this wave's 32 keys
            f32x16 s_acc, dp_acc;
            clear(s_acc);
            clear(dp_acc);
#pragma unroll
            for (int ks = 0; ks < QK_STEPS; ++ks) {
                const bf16x8 a = natural_fragment<DQK>(q_natural, 32 * qb + lq, ks, g);
                s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, kf[ks], s_acc, 0, 0, 0);
            }
#pragma unroll
            for (int ks = 0; ks < V_STEPS; ++ks) {
                const bf16x8 a = natural_fragment<DV>(do_natural, 32 * qb + lq, ks, g);
                dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, vf[ks], dp_acc, 0, 0, 0);
            }
            // lane holds key lq and queries 32*qb + 8*(i/4) + 4*g + i%4
            const bool diagonal = q0 + 32 * qb < wave_k0 + 31;
            bf16x8 pf[2], dsf[2];
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                u32x4 p_packed, ds_packed;
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int i4 = 2 * n + half;
                    const int q_local = 32 * qb + 8 * i4 + 4 * g;
                    const f32x4 lse4 = *reinterpret_cast<const f32x4*>(stats + q_local);
                    const f32x4 delta4 = *reinterpret_cast<const f32x4*>(stats + BWD_TILE + q_local);
                    float p[4], ds[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int i = 4 * i4 + e;
                        float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[i], c, -lse4[e]));
                        if (diagonal && q0 + q_local + e < key_row) probability = 0.f;
                        p[e] = probability;
                        ds[e] = probability * (dp_acc[i] - delta4[e]) * scale;
                    }
                    p_packed[2 * half] = pack_bf16(p[0], p[1]);
                    p_packed[2 * half + 1] = pack_bf16(p[2], p[3]);
                    ds_packed[2 * half] = pack_bf16(ds[0], ds[1]);
                    ds_packed[2 * half + 1] = pack_bf16(ds[2], ds[3]);
                }
                pf[n] = __builtin_bit_cast(bf16x8, p_packed);
                dsf[n] = __builtin_bit_cast(bf16x8, ds_packed);
            }
            // dV += P^T dO, dK += dS^T Q (contraction over the 32 queries)
#pragma unroll
            for (int n = 0; n < 2; ++n) {
#pragma unroll
                for (int d = 0; d < DV_BLOCKS; ++d) {
                    const bf16x8 bo = transposed_fragment<DV>(do_transposed, 32 * d + lq, 2 * qb + n, g);
                    dv_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[n], bo, dv_acc[d], 0, 0, 0);
                }
#pragma unroll
                for (int d = 0; d < DK_BLOCKS; ++d) {
                    const bf16x8 bq = transposed_fragment<DQK>(q_transposed, 32 * d + lq, 2 * qb + n, g);
                    dk_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[n], bq, dk_acc[d], 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue: lane holds column 32*d + lq and keys 8*(i/4) + 4*g + i%4
    __syncthreads();
    unsigned char* dk_lds = lds + wave * 32 * (C::DK_PITCH + C::DV_PITCH);
    unsigned char* dv_lds = dk_lds + 32 * C::DK_PITCH;
#pragma unroll
    for (int d = 0; d < DK_BLOCKS; ++d) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = 8 * (i / 4) + 4 * g + i % 4;
            const __bf16 rounded = (__bf16)dk_acc[d][i];
            *reinterpret_cast<__bf16*>(dk_lds + row * C::DK_PITCH + 2 * (32 * d + lq)) = rounded;
        }
    }
#pragma unroll
    for (int d = 0; d < DV_BLOCKS; ++d) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = 8 * (i / 4) + 4 * g + i % 4;
            const __bf16 rounded = (__bf16)dv_acc[d][i];
            *reinterpret_cast<__bf16*>(dv_lds + row * C::DV_PITCH + 2 * (32 * d + lq)) = rounded;
        }
    }
    __syncthreads();
    bf16_t* dk_base = key_gradient + ((size_t)b * S * heads + h) * DQK;
    bf16_t* dv_base = value_gradient + ((size_t)b * S * heads + h) * DV;
    for (int index = lane; index < 32 * (DQK / 8); index += 64) {
        const int row = index / (DQK / 8);
        const int chunk = index % (DQK / 8);
        if (wave_k0 + row < S) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(dk_lds + row * C::DK_PITCH + 16 * chunk);
            *reinterpret_cast<u32x4*>(dk_base + (size_t)(wave_k0 + row) * qk_stride + 8 * chunk) = bits;
        }
    }
    for (int index = lane; index < 32 * (DV / 8); index += 64) {
        const int row = index / (DV / 8);
        const int chunk = index % (DV / 8);
        if (wave_k0 + row < S) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(dv_lds + row * C::DV_PITCH + 16 * chunk);
            *reinterpret_cast<u32x4*>(dv_base + (size_t)(wave_k0 + row) * v_stride + 8 * chunk) = bits;
        }
    }
}

// ---- dQ ----------------------------------------------------------------------

template <int DQK, int DV>
struct QueryGradConfig {
    using KT = DualTile<DQK>;
    static constexpr int QUERIES = 128;  // per workgroup
    static constexpr int V_PITCH = 2 * DV + 16;
    static constexpr int V_BYTES = BWD_TILE * V_PITCH;
    static constexpr int V_CHUNKS = BWD_TILE * (DV / 8);
    static constexpr int V_PER_THREAD = V_CHUNKS / BWD_THREADS;
    static constexpr int K_NATURAL = 0;
    static constexpr int K_TRANSPOSED = K_NATURAL + KT::NATURAL_BYTES;
    static constexpr int V_NATURAL = K_TRANSPOSED + KT::TRANSPOSED_BYTES;
    static constexpr int STAGE_BYTES = V_NATURAL + V_BYTES;
    static constexpr int DQ_PITCH = 2 * DQK + 16;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static_assert(QUERIES * DQ_PITCH <= LDS_BYTES, "epilogue staging must fit");
    static_assert(V_CHUNKS % BWD_THREADS == 0, "V tile must divide evenly over the workgroup");
};

template <int DQK, int DV>
__global__ __launch_bounds__(BWD_THREADS) void attention_query_gradient_kernel(
    bf16_t* __restrict__ query_gradient, const bf16_t* __restrict__ output_gradient,
    const float* __restrict__ logsumexp, const float* __restrict__ delta, const bf16_t* __restrict__ query,
    const bf16_t* __restrict__ key, const bf16_t* __restrict__ value, int sequence_length, int heads,
    int query_blocks, float scale) {
    using C = QueryGradConfig<DQK, DV>;
    using KT = DualTile<DQK>;
    constexpr int QK_STEPS = DQK / 16;
    constexpr int V_STEPS = DV / 16;
    constexpr int DQ_BLOCKS = DQK / 32;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int S = sequence_length;

    int bh, qb_rank;
    xcd_order(blockIdx.x, gridDim.x / query_blocks, query_blocks, bh, qb_rank);
    const int qb = query_blocks - 1 - qb_rank;  // heaviest (last) query blocks first
    const int b = bh / heads;
    const int h = bh % heads;
    const int q0 = qb * C::QUERIES;
    const int wave_q0 = q0 + 32 * wave;
    const int q_row = wave_q0 + lq;
    const bool valid = q_row < S;

    const size_t qk_stride = (size_t)heads * DQK;
    const size_t v_stride = (size_t)heads * DV;
    const bf16_t* q_base = query + ((size_t)b * S * heads + h) * DQK;
    const bf16_t* k_base = key + ((size_t)b * S * heads + h) * DQK;
    const bf16_t* v_base = value + ((size_t)b * S * heads + h) * DV;
    const bf16_t* do_base = output_gradient + ((size_t)b * S * heads + h) * DV;

    // Q and dO rows of this wave as B operands (column = query lq)
    bf16x8 qf[QK_STEPS], dof[V_STEPS];
    load_row_fragments<DQK>(qf, q_base, qk_stride, q_row, valid, g);
    load_row_fragments<DV>(dof, do_base, v_stride, q_row, valid, g);
    const float lse2 = valid ? logsumexp[((size_t)b * heads + h) * S + q_row] * LOG2E : 0.f;
    const float row_delta = valid ? delta[((size_t)b * heads + h) * S + q_row] : 0.f;

    f32x16 dq_acc[DQ_BLOCKS];
#pragma unroll
    for (int d = 0; d < DQ_BLOCKS; ++d) clear(dq_acc[d]);

    const float c = scale * LOG2E;
    const int last_key = min(S, q0 + C::QUERIES) - 1;
    const int tiles = last_key / BWD_TILE + 1;

    u32x2 k_stage[KT::PER_THREAD][4];
    u32x4 v_stage[C::V_PER_THREAD];
    auto load_tile = [&](int tile) {
        const int row0 = tile * BWD_TILE;
        load_units<DQK>(k_stage, k_base, qk_stride, row0, S, tid);
#pragma unroll
        for (int i = 0; i < C::V_PER_THREAD; ++i) {
            const int id = tid + BWD_THREADS * i;
            const int row = row0 + id / (DV / 8);
            u32x4 bits = {0, 0, 0, 0};
            if (row < S) bits = *reinterpret_cast<const u32x4*>(v_base + (size_t)row * v_stride + 8 * (id % (DV / 8)));
            v_stage[i] = bits;
        }
    };
    auto store_tile = [&](int stage) {
        unsigned char* base = lds + stage * C::STAGE_BYTES;
        store_units<DQK, true, true>(k_stage, base + C::K_NATURAL, base + C::K_TRANSPOSED, tid);
#pragma unroll
        for (int i = 0; i < C::V_PER_THREAD; ++i) {
            const int id = tid + BWD_THREADS * i;
            *reinterpret_cast<u32x4*>(base + C::V_NATURAL + (id / (DV / 8)) * C::V_PITCH + 16 * (id % (DV / 8))) = v_stage[i];
        }
    };

    load_tile(0);
    store_tile(0);
    __syncthreads();
    for (int tile = 0; tile < tiles; ++tile) {
        const int stage = tile & 1;
        const bool more = tile + 1 < tiles;
        if (more) load_tile(tile + 1);
        const int key0 = tile * BWD_TILE;
        if (key0 <= wave_q0 + 31) {
            const unsigned char* base = lds + stage * C::STAGE_BYTES;
            const unsigned char* k_natural = base + C::K_NATURAL;
            const unsigned char* k_transposed = base + C::K_TRANSPOSED;
            const unsigned char* v_natural = base + C::V_NATURAL;

            f32x16 s_acc[2], dp_acc[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                clear(s_acc[mb]);
                clear(dp_acc[mb]);
            }
#pragma unroll
            for (int ks = 0; ks < QK_STEPS; ++ks) {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    const bf16x8 a = natural_fragment<DQK>(k_natural, 32 * mb + lq, ks, g);
                    s_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s_acc[mb], 0, 0, 0);
                }
            }
#pragma unroll
            for (int ks = 0; ks < V_STEPS; ++ks) {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(v_natural + (32 * mb + lq) * C::V_PITCH + 32 * ks + 16 * g);
                    dp_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, dof[ks], dp_acc[mb], 0, 0, 0);
                }
            }
            // lane holds query lq and keys key0 + 32*mb + 8*(i/4) + 4*g + i%4
            const bool diagonal = key0 + BWD_TILE - 1 > wave_q0;
            bf16x8 dsf[4];
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                u32x4 packed;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int i = 8 * (n % 2) + 2 * j;
                    float ds[2];
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[n / 2][i + e], c, -lse2));
                        const int k = key0 + 32 * (n / 2) + 8 * ((i + e) / 4) + 4 * g + (i + e) % 4;
                        if (diagonal && k > q_row) probability = 0.f;
                        ds[e] = probability * (dp_acc[n / 2][i + e] - row_delta) * scale;
                    }
                    packed[j] = pack_bf16(ds[0], ds[1]);
                }
                dsf[n] = __builtin_bit_cast(bf16x8, packed);
            }
            // dQ^T += K^T dS^T (contraction over the 64 keys)
#pragma unroll
            for (int n = 0; n < 4; ++n) {
#pragma unroll
                for (int d = 0; d < DQ_BLOCKS; ++d) {
                    const bf16x8 a = transposed_fragment<DQK>(k_transposed, 32 * d + lq, n, g);
                    dq_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, dsf[n], dq_acc[d], 0, 0, 0);
                }
            }
        }
        if (more) store_tile(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds query lq and columns 32*d + 8*(i/4) + 4*g + i%4
    unsigned char* dq_lds = lds + (32 * wave) * C::DQ_PITCH;
#pragma unroll
    for (int d = 0; d < DQ_BLOCKS; ++d) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            u32x2 packed;
            packed.x = pack_bf16(dq_acc[d][4 * i4 + 0], dq_acc[d][4 * i4 + 1]);
            packed.y = pack_bf16(dq_acc[d][4 * i4 + 2], dq_acc[d][4 * i4 + 3]);
            *reinterpret_cast<u32x2*>(dq_lds + lq * C::DQ_PITCH + 2 * (32 * d + 8 * i4 + 4 * g)) = packed;
        }
    }
    __syncthreads();
    bf16_t* dq_base = query_gradient + ((size_t)b * S * heads + h) * DQK;
    for (int index = lane; index < 32 * (DQK / 8); index += 64) {
        const int row = index / (DQK / 8);
        const int chunk = index % (DQK / 8);
        if (wave_q0 + row < S) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(dq_lds + row * C::DQ_PITCH + 16 * chunk);
            *reinterpret_cast<u32x4*>(dq_base + (size_t)(wave_q0 + row) * qk_stride + 8 * chunk) = bits;
        }
    }
}

template <typename Kernel>
void raise_lds_limit(Kernel kernel, int bytes) {
    if (bytes > 64 * 1024) {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    }
}

template <int DQK, int DV>
void launch_backward(bf16_t* query_gradient, bf16_t* key_gradient, bf16_t* value_gradient,
                     const bf16_t* output_gradient, const bf16_t* output, const float* logsumexp,
                     const bf16_t* query, const bf16_t* key, const bf16_t* value, float* delta, int batch_size,
                     int sequence_length, int heads, float scale, hipStream_t stream) {
    using KC = KeyGradConfig<DQK, DV>;
    using QC = QueryGradConfig<DQK, DV>;
    const long long rows = (long long)batch_size * sequence_length * heads;
    const long long groups = (long long)batch_size * heads;
    const int key_blocks = (sequence_length + KC::KEYS - 1) / KC::KEYS;
    const int query_blocks = (sequence_length + QC::QUERIES - 1) / QC::QUERIES;
    if ((rows + 15) / 16 > 0x7fffffffLL || groups * key_blocks > 0x7fffffffLL) {
        throw std::invalid_argument("attention backward: problem exceeds the grid limit");
    }
    static thread_local bool prepared = false;
    if (!prepared) {
        raise_lds_limit(attention_key_gradient_kernel<DQK, DV>, KC::LDS_BYTES);
        raise_lds_limit(attention_query_gradient_kernel<DQK, DV>, QC::LDS_BYTES);
        prepared = true;
    }
    hipLaunchKernelGGL((attention_delta_kernel<DV>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream, delta,
                       output_gradient, output, batch_size, sequence_length, heads);
    HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL((attention_key_gradient_kernel<DQK, DV>), dim3((unsigned)(groups * key_blocks)),
                       dim3(BWD_THREADS), KC::LDS_BYTES, stream, key_gradient, value_gradient, output_gradient,
                       logsumexp, delta, query, key, value, sequence_length, heads, key_blocks, scale);
    HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL((attention_query_gradient_kernel<DQK, DV>), dim3((unsigned)(groups * query_blocks)),
                       dim3(BWD_THREADS), QC::LDS_BYTES, stream, query_gradient, output_gradient, logsumexp, delta,
                       query, key, value, sequence_length, heads, query_blocks, scale);
    HIP_CHECK(hipGetLastError());
}

}  // namespace

void attention_backward_dispatch(bf16_t* query_gradient, bf16_t* key_gradient, bf16_t* value_gradient,
                                 const bf16_t* output_gradient, const bf16_t* output, const float* logsumexp,
                                 const bf16_t* query, const bf16_t* key, const bf16_t* value, float* delta,
                                 int batch_size, int sequence_length, int heads, int qk_head_size, int v_head_size,
                                 float scale, hipStream_t stream) {
#define DSCUDA_BWD_CASE(DQK, DV)                                                                                   \
    if (qk_head_size == DQK && v_head_size == DV) {                                                                \
        launch_backward<DQK, DV>(query_gradient, key_gradient, value_gradient, output_gradient, output, logsumexp, \
                                 query, key, value, delta, batch_size, sequence_length, heads, scale, stream);      \
        return;                                                                                                    \
    }
    DSCUDA_BWD_CASE(192, 128)
    DSCUDA_BWD_CASE(128, 128)
    DSCUDA_BWD_CASE(64, 64)
#undef DSCUDA_BWD_CASE
    throw std::invalid_argument("attention backward: unsupported head sizes (d_qk,d_v) = (" +
                                std::to_string(qk_head_size) + "," + std::to_string(v_head_size) + ")");
}

}  // namespace dscuda
