// Recompute-based causal attention backward for gfx950 (per-head K/V, the
// 128 nope + 64 rope | 128 value MLA prefill geometry and the square flash
// geometries).  The mathematics is the analytic backward the reference states
// in reference/python/mla.py:42-57 -- P = exp(S - LSE), delta = sum(dO * O),
// dS = P (dP - delta) scale -- with per-head K and V; the reference has no
// kernel for this form (its absorbed backward, kernels/attention/mla/sm89.cu:
// 295-411, is one scalar workgroup per gradient row).
//
// Three launches; every gradient row has exactly one writer (no atomics):
//
//   statistics   per query row: LSE * log2(e) and delta = sum_c dO * O, stored per
//                64-query tile (padding rows carry LSE = +inf, so they weigh nothing)
//   dK/dV        a workgroup owns 128 keys and walks the 64-query tiles from the
//                diagonal to the end:
//                    S = Q K^T, dP = dO V^T          (queries x keys)
//                    dV += P^T dO,  dK += dS^T Q
//                and leaves dS (bf16, before the scale factor) in the workspace,
//                one 16 KB block per (key block, query tile)
//   dQ           the separate accumulation pass: a plain product dQ = scale * dS K
//                over the stored dS blocks, nothing is recomputed
//
// Operand feeds.  Q and dO tiles arrive by global_load_lds and are stored once,
// row-major.  Both orientations are read from that one copy: 16-byte row reads
// give the operand of S / dP (contraction over the head dimension), and
// ds_read_b64_tr_b16 gives the operand of dV / dK (contraction over queries).
// The 16-byte chunk c of row r sits at chunk c ^ f(r); f is chosen per row
// length so that the 16-row column reads and the 4-row x 64-byte transposing
// reads are both free of bank conflicts.  P and dS leave the MFMA in its C
// layout and go back in as operands without crossing lanes.
//
// dS blocks are written exactly as the registers hold them (16 bytes per lane,
// 1 KB per wave instruction, lanes permuted by a constant XOR so that the dQ
// pass reads them back transposed without bank conflicts).
#include "attn_kernels.h"
#include "hip_common.h"
#include "index_math.h"

#include <stdexcept>
#include <string>
#include <type_traits>

namespace dscuda {
namespace {

constexpr int BWD_THREADS = 256;
constexpr int QTILE = 64;                            // queries per streamed tile
constexpr int KBLOCK = 128;                          // keys per workgroup of the dK/dV kernel
constexpr int DS_BLOCK_BYTES = KBLOCK * QTILE * 2;   // one (key block, query tile) of dS, bf16
constexpr int DS_BLOCK_FLOATS = DS_BLOCK_BYTES / 4;
constexpr int STAT_FLOATS = 2 * QTILE;               // per query tile: LSE*log2e [64], delta [64]

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4* transposing_read_pointer;

using index_math::ds_block_count;
using index_math::ds_block_index;
using index_math::tile_swizzle;

// global_load_lds with 4 bytes per lane (256 consecutive LDS bytes per wave instruction)
__device__ __forceinline__ void direct_load_4_offset(const void* uniform_base, unsigned byte_offset, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1"
                 :
                 : "v"(byte_offset), "s"(uniform_base), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory", "m0");
}

// One wave's share of the global_load_lds requests of a [64][ROW_BYTES] tile that
// WAVES waves fetch together; the offsets are those of index_math::TileRequestMath.
// Full tiles take the fast form (a per-lane base per residue, computed once, plus
// compile-time constants); at a ragged end rows past `row_limit` repeat that row
// (general form).
template <int ROW_BYTES, int WAVES>
struct TileRequests {
    using Math = index_math::TileRequestMath<ROW_BYTES, WAVES, QTILE>;
    static constexpr int LOADS = Math::LOADS;
    static constexpr int PERIOD = Math::PERIOD;
    unsigned base[PERIOD];

    __device__ __forceinline__ void init(unsigned row_stride, int wave, int lane) {
#pragma unroll
        for (int r = 0; r < PERIOD; ++r) base[r] = Math::base_of(r, lane, row_stride, wave);
    }
    // `tile` = address of the tile's first row (uniform)
    __device__ __forceinline__ void request(const unsigned char* tile, unsigned row_stride, int row_limit,
                                            unsigned lds_target, int wave) const {
        if (row_limit >= QTILE - 1) {
            const unsigned char* rows = tile + (size_t)Math::rows_before(0, wave) * row_stride;
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                direct_load_16_offset(rows + (size_t)Math::rows_before(i, 0) * row_stride,
                                      Math::lane_part(base[i % PERIOD], i), lds_target + (wave * LOADS + i) * 1024);
            }
        } else {
            const int lane = fresh_lane_id();
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                direct_load_16_offset(tile, Math::offset_of(wave * LOADS + i, lane, row_stride, row_limit),
                                      lds_target + (wave * LOADS + i) * 1024);
            }
        }
    }
};

// Per-lane byte offsets of the fragment reads of a row-major swizzled tile
// (index_math::TileReadMath); a user adds the (run-time) tile base to the per-lane
// values once per tile.
template <int ROW_BYTES>
struct TileReads {
    using Math = index_math::TileReadMath<ROW_BYTES>;
    static constexpr int NAT = Math::NAT;
    static constexpr int TR = Math::TR;
    unsigned natural[NAT];
    unsigned transposed[2][TR];

    __device__ __forceinline__ void init(int lane) {
#pragma unroll
        for (int i = 0; i < NAT; ++i) natural[i] = Math::natural(i, lane);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < TR; ++i) transposed[h][i] = Math::transposed(h, i, lane);
        }
    }
};

// `at` = TileReads::natural plus the tile's LDS offset; rows ROW0 + lane%32, k-step KS
template <int ROW_BYTES, int ROW0, int KS>
__device__ __forceinline__ bf16x8 natural_fragment(const unsigned char* lds, const unsigned (&at)[TileReads<ROW_BYTES>::NAT]) {
    using Math = index_math::TileReadMath<ROW_BYTES>;
    return *reinterpret_cast<const bf16x8*>(lds + at[KS % Math::NAT] + Math::natural_constant(ROW0, KS));
}

// `at` = TileReads::transposed plus the tile's LDS offset; 16 rows from ROW0, column block BLOCK
template <int ROW_BYTES, int ROW0, int BLOCK>
__device__ __forceinline__ bf16x8 transposed_fragment(const unsigned char* lds,
                                                      const unsigned (&at)[2][TileReads<ROW_BYTES>::TR]) {
    using Math = index_math::TileReadMath<ROW_BYTES>;
    constexpr int CONSTANT = Math::transposed_constant(ROW0, BLOCK);
    const s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (transposing_read_pointer)(lds + at[0][BLOCK % Math::TR] + CONSTANT));
    const s16x4 high = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (transposing_read_pointer)(lds + at[1][BLOCK % Math::TR] + CONSTANT));
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
}

// f(integral_constant<int, BEGIN>) ... f(integral_constant<int, END - 1>)
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// at = reads + offset, as values the optimiser cannot take apart again: the
// fragment reads then keep the form (per-lane register) + (immediate) instead of
// one address computation per read.
__device__ __forceinline__ unsigned opaque(unsigned value) {
    asm volatile("" : "+v"(value));
    return value;
}
template <int N>
__device__ __forceinline__ void rebase(unsigned (&at)[N], const unsigned (&reads)[N], unsigned offset) {
#pragma unroll
    for (int i = 0; i < N; ++i) at[i] = opaque(reads[i] + offset);
}
template <int N>
__device__ __forceinline__ void rebase(unsigned (&at)[2][N], const unsigned (&reads)[2][N], unsigned offset) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int i = 0; i < N; ++i) at[h][i] = opaque(reads[h][i] + offset);
    }
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

// ---- statistics ---------------------------------------------------------------

// One 16-lane group per (b, s, h) row of the sequence padded to whole query tiles.
template <int DV>
__global__ __launch_bounds__(256) void attention_backward_statistics_kernel(
    float* __restrict__ statistics, const bf16_t* __restrict__ output_gradient, const bf16_t* __restrict__ output,
    const float* __restrict__ logsumexp, int batch_size, int sequence_length, int heads, int query_tiles) {
    const long long padded = (long long)query_tiles * QTILE;
    const long long rows = (long long)batch_size * padded * heads;
    const long long row = (long long)blockIdx.x * 16 + threadIdx.x / 16;
    const int part = threadIdx.x % 16;
    if (row >= rows) {
        return;
    }
    const long long h = row % heads;
    const long long s = (row / heads) % padded;
    const long long b = row / (heads * padded);
    float sum = 0.f;
    float lse2 = INFINITY;
    if (s < sequence_length) {
        const long long source = ((b * sequence_length + s) * heads + h) * DV;
#pragma unroll
        for (int c = part * 8; c < DV; c += 128) {
            const u32x4 x = *reinterpret_cast<const u32x4*>(output_gradient + source + c);
            const u32x4 y = *reinterpret_cast<const u32x4*>(output + source + c);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sum += bf16_bits_to_float(x[j] & 0xffffu) * bf16_bits_to_float(y[j] & 0xffffu);
                sum += bf16_bits_to_float(x[j] >> 16) * bf16_bits_to_float(y[j] >> 16);
            }
        }
        lse2 = logsumexp[(b * heads + h) * sequence_length + s] * LOG2E;
    }
#pragma unroll
    for (int offset = 1; offset < 16; offset <<= 1) sum += __shfl_xor(sum, offset);
    if (part == 0) {
        float* target = statistics + ((b * heads + h) * query_tiles + s / QTILE) * STAT_FLOATS + s % QTILE;
        target[0] = lse2;
        target[QTILE] = sum;
    }
}

// ---- dK / dV (and dS) -----------------------------------------------------------
//
// Eight waves, two per SIMD.  Waves g and g + 4 (g = 0..3, the same SIMD) share the
// 32 keys of group g and split the work of a tile by product:
//
//   value wave (g)      S = Q K^T (K rows in registers)  ->  P = exp2(S c - LSE)
//                       ->  dV += P^T dO;  P goes to the key wave through LDS
//   key wave (g + 4)    dP = dO V^T (V rows in registers)  ->  dS = P (dP - delta)
//                       ->  dK += dS^T Q;  dS goes to the workspace
//
// The two waves of a SIMD run different instruction streams, so while one wave
// forms probabilities the other feeds the matrix pipeline.  Two workgroup barriers
// per tile keep the pair, the tile stages and the P hand-over in step:
//
//   barrier A   value wave: P(i) -> LDS               key wave: dP(i)
//   barrier B   value wave: dV(i), S(i+1)            key wave: dS(i), dK(i)
//
// so that in either phase one wave of a SIMD has vector work while the other has
// matrix work.  Tile i lives in stage i % 3 and is requested two tiles ahead; it is
// complete one phase before its first use.

constexpr int KV_THREADS = 512;

template <int DQK, int DV>
struct KeyValueGradConfig {
    static constexpr int Q_ROW = 2 * DQK;
    static constexpr int O_ROW = 2 * DV;
    static constexpr int Q_BYTES = QTILE * Q_ROW;
    static constexpr int O_BYTES = QTILE * O_ROW;
    static constexpr int STAT_BYTES = STAT_FLOATS * 4;
    static constexpr int STAGE_BYTES = Q_BYTES + O_BYTES + STAT_BYTES;
    static constexpr int STAGES = 3;
    static constexpr int P_BYTES = QTILE * 32 * 2;                  // P of one tile and key group, bf16
    static constexpr int HANDOVER_AT = STAGES * STAGE_BYTES;
    static constexpr int LDS_BYTES = HANDOVER_AT + 4 * P_BYTES;   // one buffer per key group
    static constexpr int DK_PITCH = 2 * DQK;   // epilogue staging
    static constexpr int DV_PITCH = 2 * DV;
    static_assert(4 * 32 * (DK_PITCH + DV_PITCH) <= HANDOVER_AT, "epilogue staging must fit");
    static_assert(LDS_BYTES <= 160 * 1024, "stages must fit the LDS");
};

template <int DQK, int DV>
__global__ __launch_bounds__(KV_THREADS) void attention_key_value_gradient_kernel(
    bf16_t* __restrict__ key_gradient, bf16_t* __restrict__ value_gradient, unsigned char* __restrict__ ds_blocks,
    const float* __restrict__ statistics, const bf16_t* __restrict__ output_gradient,
    const bf16_t* __restrict__ query, const bf16_t* __restrict__ key, const bf16_t* __restrict__ value,
    int sequence_length, int heads, int kv_heads, int key_blocks, int query_tiles, int first_pair, float scale) {
    using C = KeyValueGradConfig<DQK, DV>;
    constexpr int QK_STEPS = DQK / 16;
    constexpr int V_STEPS = DV / 16;
    constexpr int DK_BLOCKS = DQK / 32;
    constexpr int DV_BLOCKS = DV / 32;
    constexpr int WAVES = KV_THREADS / 64;
    constexpr int RING = 4;   // fragments read ahead of the MFMA that takes them

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const bool key_wave = wave >= 4;
    const int group = wave % 4;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int S = sequence_length;

    // Work order.  The key blocks of a (batch, head) pair all stream the same query
    // tiles, so they are kept together: pairs are dealt to the XCDs (private L2s), one
    // pair at a time per XCD, key block 0 (which sees every query: the heaviest) first.
    // Every key block walks the tiles from the last one down to its diagonal: blocks
    // started together then read the same tile at the same time, and one fetch from
    // memory serves them all.
    int bh, kb;
    {
        constexpr int XCDS = 8;
        const int pairs = gridDim.x / key_blocks;
        if (pairs % XCDS == 0) {
            const int slot = blockIdx.x / XCDS;
            bh = blockIdx.x % XCDS + XCDS * (slot / key_blocks);
            kb = slot % key_blocks;
        } else {
            bh = blockIdx.x / key_blocks;
            kb = blockIdx.x % key_blocks;
        }
    }
    // The launch covers the (batch, key/value head) pairs first_pair .. first_pair + gridDim.x / key_blocks - 1.
    // `heads` query heads share `kv_heads` key/value heads: query heads h * sharing .. + sharing - 1 read key/value
    // head h, and this workgroup walks the query tiles of each of them in turn, all into the same dK / dV
    // accumulators.  The dS blocks of member m of pair first_pair + i sit at position i * sharing + m of the
    // workspace (query-head order, which is how the query-gradient pass finds them).
    const int sharing = heads / kv_heads;
    const int local_pair = bh;
    bh += first_pair;
    const int b = bh / kv_heads;
    const int h = bh % kv_heads;          // key/value head
    const int first_query_head = h * sharing;
    const int k0 = kb * KBLOCK;
    const int group_k0 = k0 + 32 * group;
    const int key_row = group_k0 + lq;

    const size_t qk_stride = (size_t)kv_heads * DQK;   // rows of K and dK
    const size_t v_stride = (size_t)kv_heads * DV;     // rows of V and dV
    const unsigned q_stride_bytes = (unsigned)heads * DQK * 2;
    const unsigned o_stride_bytes = (unsigned)heads * DV * 2;
    // of the first query head of the group; member m follows m head rows further
    const unsigned char* q_base =
        reinterpret_cast<const unsigned char*>(query + ((size_t)b * S * heads + first_query_head) * DQK);
    const unsigned char* do_base =
        reinterpret_cast<const unsigned char*>(output_gradient + ((size_t)b * S * heads + first_query_head) * DV);
    const float* stat_base = statistics + ((size_t)b * heads + first_query_head) * query_tiles * STAT_FLOATS;
    const unsigned lds_base = lds_offset_of(lds);

    // Step `index` of the walk works on tile query_tiles - 1 - index % tiles of member index / tiles.
    const int tiles = query_tiles - 2 * kb;   // >= 1, per member
    const int steps = tiles * sharing;

    // Tiles are requested by the four value waves, each the same number of loads per
    // tile: a value wave then knows that all but its last REQUEST_LOADS loads have
    // landed, and the key waves' vector-memory counter only ever holds their dS
    // stores, which nothing has to wait for.
    TileRequests<C::Q_ROW, 4> q_requests;
    TileRequests<C::O_ROW, 4> o_requests;
    q_requests.init(q_stride_bytes, wave % 4, lane);
    o_requests.init(o_stride_bytes, wave % 4, lane);
    constexpr int REQUEST_LOADS = TileRequests<C::Q_ROW, 4>::LOADS + TileRequests<C::O_ROW, 4>::LOADS + 1;
    // step `index` = tile-step `local` of member `member` (the callers keep the three in step: no division here)
    auto request_tile = [&](int index, int member, int local) {
        const int tile = query_tiles - 1 - local;
        const int row0 = tile * QTILE;
        const int row_limit = S - 1 - row0;
        const unsigned target = lds_base + (index % 3) * C::STAGE_BYTES;
        q_requests.request(q_base + (size_t)member * (DQK * 2) + (size_t)row0 * q_stride_bytes, q_stride_bytes, row_limit,
                           target, wave);
        o_requests.request(do_base + (size_t)member * (DV * 2) + (size_t)row0 * o_stride_bytes, o_stride_bytes, row_limit,
                           target + C::Q_BYTES, wave);
        // statistics: 128 floats = two loads; waves 2 and 3 repeat those of waves 0 and 1
        // (same bytes to the same place) so that every value wave issues the same count
        direct_load_4_offset(stat_base + ((size_t)member * query_tiles + tile) * STAT_FLOATS + 64 * (wave % 2), 4u * lane,
                             target + C::Q_BYTES + C::O_BYTES + 256 * (wave % 2));
    };

    // per-lane read offsets inside a stage
    TileReads<C::Q_ROW> q_reads;
    TileReads<C::O_ROW> o_reads;
    q_reads.init(lane);
    o_reads.init(lane);
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // hand-over buffer of this key group: P as the value wave's registers hold it,
    // piece (query half, 16-query step) of 1 KB, 16 bytes per lane
    const unsigned handover = C::HANDOVER_AT + group * C::P_BYTES + 16 * lane;

    if (!key_wave) {
        // ================= value wave: S, P, dV =================
        request_tile(0, 0, 0);
        if (steps > 1) {
            if (tiles > 1) request_tile(1, 0, 1); else request_tile(1, 1, 0);
        }
        const bf16_t* k_base = key + ((size_t)b * S * kv_heads + h) * DQK;
        bf16x8 kf[QK_STEPS];   // B operand: column = key lq
        load_row_fragments<DQK>(kf, k_base, qk_stride, key_row, key_row < S, g);
        f32x16 dv_acc[DV_BLOCKS];
#pragma unroll
        for (int d = 0; d < DV_BLOCKS; ++d) clear(dv_acc[d]);
        const float c = scale * LOG2E;
        constexpr int S_MFMAS = 2 * QK_STEPS;
        constexpr int DV_MFMAS = 4 * DV_BLOCKS;
        static_assert(RING <= DV_MFMAS && RING <= S_MFMAS, "a ring of fragments must fit each product");
        bf16x8 ring[RING];
        // S fragment K: k-step K/2 of query half K%2; dV fragment K: 16-query step K / DV_BLOCKS, column block K % DV_BLOCKS
        auto s_fragment = [&](const unsigned (&q_at)[TileReads<C::Q_ROW>::NAT], auto k_tag) -> bf16x8 {
            constexpr int K = decltype(k_tag)::value;
            return natural_fragment<C::Q_ROW, 32 * (K % 2), K / 2>(lds, q_at);
        };
        auto dv_fragment = [&](const unsigned (&o_at)[2][TileReads<C::O_ROW>::TR], auto k_tag) -> bf16x8 {
            constexpr int K = decltype(k_tag)::value;
            return transposed_fragment<C::O_ROW, 16 * (K / DV_BLOCKS), K % DV_BLOCKS>(lds, o_at);
        };
        // S of tile `index` (both query halves: two independent accumulation chains),
        // fragments through the ring; the tail reads the statistics of the tile's queries.
        f32x16 s_acc[2];
        f32x4 lse4[2][4];   // queries 32*qb + 8*i4 + 4*g + (0..3)
        auto score_stream = [&](int index) {
            const unsigned stage = (index % 3) * C::STAGE_BYTES;
            unsigned q_at[TileReads<C::Q_ROW>::NAT];
            rebase(q_at, q_reads.natural, stage);
            const unsigned stats_at = opaque(stage + C::Q_BYTES + C::O_BYTES + 16 * g);
            static_for<0, RING>([&](auto k_tag) { ring[decltype(k_tag)::value] = s_fragment(q_at, k_tag); });
            static_for<0, S_MFMAS>([&](auto k_tag) {
                constexpr int K = decltype(k_tag)::value;
                constexpr int KS = K / 2;
                s_acc[K % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[K % RING], kf[KS],
                                                                       KS == 0 ? zero : s_acc[K % 2], 0, 0, 0);
                if constexpr (K + RING < S_MFMAS) {
                    ring[K % RING] = s_fragment(q_at, std::integral_constant<int, K + RING>{});
                }
                if constexpr (K >= S_MFMAS - 8) {
                    constexpr int J = K - (S_MFMAS - 8);
                    lse4[J / 4][J % 4] = *reinterpret_cast<const f32x4*>(lds + stats_at + 4 * (32 * (J / 4) + 8 * (J % 4)));
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        };

        // One tile, in two phases separated by barriers:
        //   after barrier A   P of the tile from its scores (formed one phase earlier) -> hand-over
        //   after barrier B   dV of the tile, then the scores of the next tile
        // so that in either phase one wave of the SIMD has vector work and the other
        // matrix work.  MASKED applies the causal mask: it can only bite in the two
        // tiles at the diagonal, the last ones of the walk (and all the tiles a ragged
        // last block has).
        auto value_tile = [&](auto masked_tag, int index, int member, int local) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            workgroup_barrier();   // A: every wave has left tile index - 1
            if (index + 2 < steps) {
                int ahead_member = member, ahead_local = local + 2;
                while (ahead_local >= tiles) {
                    ahead_local -= tiles;
                    ++ahead_member;
                }
                request_tile(index + 2, ahead_member, ahead_local);
            }
            // P: lane holds key lq and queries 32*qb + 8*i4 + 4*g + e.  A query with
            // local index below `threshold` lies before this lane's key.
            u32x4 pf[2][2];
            const int threshold = key_row - 4 * g - (query_tiles - 1 - local) * QTILE;
            static_for<0, 2>([&](auto qb_tag) {
                constexpr int QB = decltype(qb_tag)::value;
                static_for<0, 4>([&](auto i4_tag) {
                    constexpr int I4 = decltype(i4_tag)::value;
                    float p[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        p[e] = __builtin_amdgcn_exp2f(fmaf(s_acc[QB][4 * I4 + e], c, -lse4[QB][I4][e]));
                    }
                    if constexpr (MASKED) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (32 * QB + 8 * I4 + e < threshold) p[e] = 0.f;
                        }
                    }
                    pf[QB][I4 / 2][2 * (I4 % 2)] = pack_bf16(p[0], p[1]);
                    pf[QB][I4 / 2][2 * (I4 % 2) + 1] = pack_bf16(p[2], p[3]);
                });
            });
            // hand P to the key wave
            static_for<0, 4>([&](auto piece_tag) {
                constexpr int PIECE = decltype(piece_tag)::value;
                *reinterpret_cast<u32x4*>(lds + handover + PIECE * 1024) = pf[PIECE / 2][PIECE % 2];
            });
            // this wave's share of tile index + 1 has landed (the request of tile index + 2,
            // if there is one, may stay in flight)
            if (index + 2 < steps) {
                wait_vector_memory<REQUEST_LOADS>();
            } else {
                wait_vector_memory<0>();
            }
            workgroup_barrier();   // B: P is visible, and so is all of tile index + 1

            // dV += P^T dO (contraction over the tile's 64 queries)
            const unsigned stage = (index % 3) * C::STAGE_BYTES;
            unsigned o_at[2][TileReads<C::O_ROW>::TR];
            rebase(o_at, o_reads.transposed, stage + C::Q_BYTES);
            static_for<0, RING>([&](auto k_tag) { ring[decltype(k_tag)::value] = dv_fragment(o_at, k_tag); });
            static_for<0, DV_MFMAS>([&](auto k_tag) {
                constexpr int K = decltype(k_tag)::value;
                constexpr int STEP = K / DV_BLOCKS;   // 16-query step
                constexpr int D = K % DV_BLOCKS;
                dv_acc[D] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, pf[STEP / 2][STEP % 2]),
                                                                    ring[K % RING], dv_acc[D], 0, 0, 0);
                if constexpr (K + RING < DV_MFMAS) {
                    ring[K % RING] = dv_fragment(o_at, std::integral_constant<int, K + RING>{});
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if (index + 1 < steps) {
                score_stream(index + 1);
            }
        };
        // tile 0 has landed for everybody; its scores
        wait_vector_memory<0>();
        workgroup_barrier();
        score_stream(0);
        for (int member = 0, index = 0; member < sharing; ++member) {
            for (int local = 0; local < tiles - 2; ++local, ++index) {
                value_tile(std::false_type{}, index, member, local);
            }
            for (int local = max(tiles - 2, 0); local < tiles; ++local, ++index) {
                value_tile(std::true_type{}, index, member, local);
            }
        }

        // ---- epilogue: lane holds column 32*d + lq and keys 8*(i/4) + 4*g + i%4
        __syncthreads();
        unsigned char* dv_lds = lds + group * 32 * (C::DK_PITCH + C::DV_PITCH) + 32 * C::DK_PITCH;
#pragma unroll
        for (int d = 0; d < DV_BLOCKS; ++d) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = 8 * (i / 4) + 4 * g + i % 4;
                *reinterpret_cast<__bf16*>(dv_lds + row * C::DV_PITCH + 2 * (32 * d + lq)) = (__bf16)dv_acc[d][i];
            }
        }
        __syncthreads();
        bf16_t* dv_base = value_gradient + ((size_t)b * S * kv_heads + h) * DV;
        for (int position = lane; position < 32 * (DV / 8); position += 64) {
            const int row = position / (DV / 8);
            const int chunk = position % (DV / 8);
            if (group_k0 + row < S) {
                const u32x4 bits = *reinterpret_cast<const u32x4*>(dv_lds + row * C::DV_PITCH + 16 * chunk);
                *reinterpret_cast<u32x4*>(dv_base + (size_t)(group_k0 + row) * v_stride + 8 * chunk) = bits;
            }
        }
    } else {
        // ================= key wave: dP, dS, dK =================
        const bf16_t* v_base = value + ((size_t)b * S * kv_heads + h) * DV;
        bf16x8 vf[V_STEPS];   // B operand: column = key lq
        load_row_fragments<DV>(vf, v_base, v_stride, key_row, key_row < S, g);
        f32x16 dk_acc[DK_BLOCKS];
#pragma unroll
        for (int d = 0; d < DK_BLOCKS; ++d) clear(dk_acc[d]);
        const size_t ds_head_bytes = (size_t)ds_block_count(key_blocks, query_tiles) * DS_BLOCK_BYTES;
        unsigned char* ds_group = ds_blocks + (size_t)local_pair * sharing * ds_head_bytes;   // member m: + m * ds_head_bytes
        constexpr int DK_MFMAS = 4 * DK_BLOCKS;
        constexpr int DP_MFMAS = 2 * V_STEPS;
        static_assert(RING <= DK_MFMAS && RING <= DP_MFMAS, "a ring of fragments must fit each product");
        bf16x8 ring[RING];
        // dK fragment K: 16-query step K / DK_BLOCKS, column block K % DK_BLOCKS; dP fragment K: k-step K/2 of query half K%2
        auto dk_fragment = [&](const unsigned (&q_at)[2][TileReads<C::Q_ROW>::TR], auto k_tag) -> bf16x8 {
            constexpr int K = decltype(k_tag)::value;
            return transposed_fragment<C::Q_ROW, 16 * (K / DK_BLOCKS), K % DK_BLOCKS>(lds, q_at);
        };
        auto dp_fragment = [&](const unsigned (&o_at)[TileReads<C::O_ROW>::NAT], auto k_tag) -> bf16x8 {
            constexpr int K = decltype(k_tag)::value;
            return natural_fragment<C::O_ROW, 32 * (K % 2), K / 2>(lds, o_at);
        };
        // per-lane part of the dS store addresses: slot (lane ^ (4g + 8n)) of the 1 KB
        // piece (group, qb, n) of the tile's block
        unsigned ds_slot[2];
        ds_slot[0] = group * 4096 + 16 * (lane ^ (4 * g));
        ds_slot[1] = group * 4096 + 1024 + 16 * (lane ^ (4 * g + 8));
        wait_vector_memory<0>();   // the V rows
        workgroup_barrier();       // tile 0 has landed

        for (int index = 0, member = 0, local = 0; index < steps; ++index, ++local) {
            if (local == tiles) {
                local = 0;
                ++member;
            }
            workgroup_barrier();   // A: every wave has left tile index - 1 (tile `index` landed a phase ago)
            const unsigned stage = (index % 3) * C::STAGE_BYTES;
            unsigned o_at[TileReads<C::O_ROW>::NAT], q_at[2][TileReads<C::Q_ROW>::TR];
            rebase(o_at, o_reads.natural, stage + C::Q_BYTES);
            const unsigned stats_at = opaque(stage + C::Q_BYTES + C::O_BYTES + 16 * g + 4 * QTILE);

            // dP of both query halves; the tail reads the first dK fragments and the
            // tile's delta values ahead
            f32x16 dp_acc[2];
            f32x4 delta4[2][4];   // queries 32*qb + 8*i4 + 4*g + (0..3)
            static_for<0, RING>([&](auto k_tag) { ring[decltype(k_tag)::value] = dp_fragment(o_at, k_tag); });
            rebase(q_at, q_reads.transposed, stage);
            static_for<0, DP_MFMAS>([&](auto k_tag) {
                constexpr int K = decltype(k_tag)::value;
                constexpr int KS = K / 2;
                dp_acc[K % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[K % RING], vf[KS],
                                                                        KS == 0 ? zero : dp_acc[K % 2], 0, 0, 0);
                if constexpr (K + RING < DP_MFMAS) {
                    ring[K % RING] = dp_fragment(o_at, std::integral_constant<int, K + RING>{});
                } else {
                    ring[K % RING] = dk_fragment(q_at, std::integral_constant<int, K + RING - DP_MFMAS>{});
                }
                if constexpr (K >= DP_MFMAS - 8) {
                    constexpr int J = K - (DP_MFMAS - 8);
                    delta4[J / 4][J % 4] = *reinterpret_cast<const f32x4*>(lds + stats_at + 4 * (32 * (J / 4) + 8 * (J % 4)));
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            workgroup_barrier();   // B: P of this tile is in the hand-over buffer

            // dS = P (dP - delta): lane holds key lq and queries 32*qb + 8*i4 + 4*g + e
            u32x4 packed[4];      // pieces (query half, 16-query step)
            static_for<0, 4>([&](auto piece_tag) {
                constexpr int PIECE = decltype(piece_tag)::value;
                packed[PIECE] = *reinterpret_cast<const u32x4*>(lds + handover + PIECE * 1024);
            });
            unsigned char* block = ds_group + member * ds_head_bytes +
                (size_t)ds_block_index(kb, query_tiles - 1 - local, query_tiles) * DS_BLOCK_BYTES;
            u32x4 dsf[2][2];
            static_for<0, 4>([&](auto piece_tag) {
                constexpr int PIECE = decltype(piece_tag)::value;
                constexpr int QB = PIECE / 2;
                constexpr int N = PIECE % 2;
                static_for<0, 2>([&](auto half_tag) {
                    constexpr int HALF = decltype(half_tag)::value;
                    constexpr int I4 = 2 * N + HALF;
                    float ds[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t pair = packed[PIECE][2 * HALF + e / 2];
                        const float p = (e % 2) ? __uint_as_float(pair & 0xffff0000u) : __uint_as_float(pair << 16);
                        ds[e] = p * (dp_acc[QB][4 * I4 + e] - delta4[QB][I4][e]);
                    }
                    dsf[QB][N][2 * HALF] = pack_bf16(ds[0], ds[1]);
                    dsf[QB][N][2 * HALF + 1] = pack_bf16(ds[2], ds[3]);
                });
                // written once, read by the next kernel: kept out of the way of the tiles other workgroups re-read
                __builtin_nontemporal_store(dsf[QB][N], reinterpret_cast<u32x4*>(block + (ds_slot[N] + QB * 2048)));
            });
            // dK += dS^T Q
            static_for<0, DK_MFMAS>([&](auto k_tag) {
                constexpr int K = decltype(k_tag)::value;
                constexpr int STEP = K / DK_BLOCKS;
                constexpr int D = K % DK_BLOCKS;
                dk_acc[D] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, dsf[STEP / 2][STEP % 2]),
                                                                    ring[(K + DP_MFMAS) % RING], dk_acc[D], 0, 0, 0);
                if constexpr (K + RING < DK_MFMAS) {
                    ring[(K + DP_MFMAS) % RING] = dk_fragment(q_at, std::integral_constant<int, K + RING>{});
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        }

        // ---- epilogue: lane holds column 32*d + lq and keys 8*(i/4) + 4*g + i%4
        __syncthreads();
        unsigned char* dk_lds = lds + group * 32 * (C::DK_PITCH + C::DV_PITCH);
#pragma unroll
        for (int d = 0; d < DK_BLOCKS; ++d) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = 8 * (i / 4) + 4 * g + i % 4;
                *reinterpret_cast<__bf16*>(dk_lds + row * C::DK_PITCH + 2 * (32 * d + lq)) = (__bf16)(dk_acc[d][i] * scale);
            }
        }
        __syncthreads();
        bf16_t* dk_base = key_gradient + ((size_t)b * S * kv_heads + h) * DQK;
        for (int position = lane; position < 32 * (DQK / 8); position += 64) {
            const int row = position / (DQK / 8);
            const int chunk = position % (DQK / 8);
            if (group_k0 + row < S) {
                const u32x4 bits = *reinterpret_cast<const u32x4*>(dk_lds + row * C::DK_PITCH + 16 * chunk);
                *reinterpret_cast<u32x4*>(dk_base + (size_t)(group_k0 + row) * qk_stride + 8 * chunk) = bits;
            }
        }
    }
}

// ---- dQ -------------------------------------------------------------------------

template <int DQK>
struct QueryGradConfig {
    static constexpr int QUERIES = 2 * QTILE;            // per workgroup: two query tiles
    static constexpr int STEP_KEYS = 64;                 // keys per step: half a dS block
    static constexpr int K_ROW = 2 * DQK;
    static constexpr int K_BYTES = STEP_KEYS * K_ROW;
    static constexpr int DS_HALF = DS_BLOCK_BYTES / 2;   // 64 keys x 64 queries
    static constexpr int STAGE_BYTES = K_BYTES + 2 * DS_HALF;
    static constexpr int STAGES = 3;
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int D_BLOCKS = DQK / 64;            // 32-column blocks per wave
    static_assert(LDS_BYTES <= 160 * 1024, "stages must fit the LDS");
    static_assert(4 * D_BLOCKS * 2 * 16 * 64 * 4 <= LDS_BYTES, "the final sums must fit the LDS");
    static_assert(2 * QTILE * (2 * DQK + 16) <= LDS_BYTES, "the staged gradient rows must fit the LDS");
};

// dQ^T (d x queries) = sum over keys of K^T (d x keys) dS^T (keys x queries).
// Eight waves, two per SIMD: wave w owns query tile w%2 of the workgroup's two, the
// 32-column blocks 2*d + (w/2)%2, and the 16-key steps 2*(w/4), 2*(w/4)+1 of every
// 64-key step; the two key halves are added through LDS at the end.  The pass is
// bound by the dS stream from memory: steps are requested two ahead and a wave only
// waits for the older of its two requests in flight.
constexpr int DQ_THREADS = 512;

template <int DQK>
__global__ __launch_bounds__(DQ_THREADS) void attention_query_gradient_kernel(
    bf16_t* __restrict__ query_gradient, const unsigned char* __restrict__ ds_blocks, const bf16_t* __restrict__ key,
    int sequence_length, int heads, int kv_heads, int query_blocks, int key_blocks, int query_tiles, int first_pair,
    float scale) {
    using C = QueryGradConfig<DQK>;
    constexpr int WAVES = DQ_THREADS / 64;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int S = sequence_length;

    int bh, rank;
    xcd_order(blockIdx.x, gridDim.x / query_blocks, query_blocks, bh, rank);
    // the heads in the reverse of the order in which the first pass wrote their dS blocks: what it wrote last is
    // still in the memory-side cache
    bh = gridDim.x / query_blocks - 1 - bh;
    const int jb = query_blocks - 1 - rank;   // heaviest (last) query blocks first
    const int local_pair = bh;                // position of this pair's dS blocks in the workspace
    bh += first_pair;
    const int b = bh / heads;
    const int h = bh % heads;
    const int tile_of_wave = wave % 2;
    const int column_half = (wave / 2) % 2;
    const int key_half = wave / 4;

    // query head h reads key/value head h / (heads / kv_heads)
    const unsigned k_stride_bytes = (unsigned)kv_heads * DQK * 2;
    const unsigned char* k_base =
        reinterpret_cast<const unsigned char*>(key + ((size_t)b * S * kv_heads + h / (heads / kv_heads)) * DQK);
    const unsigned char* ds_head = ds_blocks + (size_t)local_pair * ds_block_count(key_blocks, query_tiles) * DS_BLOCK_BYTES;
    const unsigned lds_base = lds_offset_of(lds);

    // query tiles of this workgroup (the second may not exist at a ragged end: it
    // then repeats the first, and its rows are not stored)
    int tile_index[2];
    tile_index[0] = 2 * jb;
    tile_index[1] = min(2 * jb + 1, query_tiles - 1);

    const int steps = 2 * (jb + 1);   // 64-key steps up to the end of key block jb
    TileRequests<C::K_ROW, WAVES> k_requests;
    k_requests.init(k_stride_bytes, wave, lane);
    constexpr int DS_LOADS = 2 * C::DS_HALF / 1024 / WAVES;   // 1 KB pieces of the two query tiles' halves per wave
    constexpr int STEP_LOADS = TileRequests<C::K_ROW, WAVES>::LOADS + DS_LOADS;
    auto request_step = [&](int step, int stage) {
        const int kb = step / 2;
        const int half = step % 2;
        const int row0 = kb * KBLOCK + half * C::STEP_KEYS;
        const unsigned target = lds_base + stage * C::STAGE_BYTES;
        // rows past the end of the sequence repeat the last one: their dS is zero
        k_requests.request(k_base + (size_t)min(row0, S - 1) * k_stride_bytes, k_stride_bytes, max(S - 1 - row0, 0),
                           target, wave);
#pragma unroll
        for (int i = 0; i < DS_LOADS; ++i) {
            const int load = DS_LOADS * wave + i;   // 16 pieces of 1 KB: two query tiles x 8
            const int t = load / 8;
            const int part = load % 8;
            const unsigned char* block =
                ds_head + (size_t)ds_block_index(kb, tile_index[t], query_tiles) * DS_BLOCK_BYTES + half * C::DS_HALF;
            direct_load_16_offset_streaming(block, (unsigned)(part * 1024 + lane * 16),
                                            target + C::K_BYTES + t * C::DS_HALF + part * 1024);
        }
    };

    f32x16 dq_acc[C::D_BLOCKS][2];
#pragma unroll
    for (int d = 0; d < C::D_BLOCKS; ++d) {
        clear(dq_acc[d][0]);
        clear(dq_acc[d][1]);
    }

    // K^T operand (ds_read_b64_tr_b16 on the row-major K rows).  A wave's column
    // blocks are 2*d + column_half, so the swizzle-dependent part of the address
    // (block % TR) is fixed per wave up to d, and the rest is an immediate.  The
    // wave's key half (32 rows down) is folded into the per-lane part as well.
    constexpr int TR = TileReads<C::K_ROW>::TR;
    constexpr int SEL = TR / 2;
    unsigned k_reads[2][SEL];
    {
        TileReads<C::K_ROW> reads;
        reads.init(lane);
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
            for (int j = 0; j < SEL; ++j) {
                k_reads[h2][j] = (column_half ? reads.transposed[h2][2 * j + 1] : reads.transposed[h2][2 * j]) +
                                 key_half * 32 * C::K_ROW;
            }
        }
    }
    // dS^T operand: column = query 32*qb + lane%32 of the tile, k = keys {4g.., 8+4g..}
    // of a 16-key step; the bytes sit where the dK/dV kernel's lanes put them.  Lane s
    // of a 16-lane group fetches the 8 bytes that hold queries 4*(s%4).. of key s/4
    // (+8 for the second read): slot ((key%32 + 32*g') ^ (4*g' + 8*n)) of the 1 KB piece
    // (key/32, qb, n), n = (lane/16)%2, g' = s%2, second half of the slot if (s%4)/2.
    // The wave's key half selects key/32.
    unsigned ds_reads[2];
    {
        const int s = lane % 16;
        const int n = (lane / 16) % 2;
        const int gp = s % 2;
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            const int slot = s / 4 + 4 * (g ^ gp) + 8 * (h2 ^ n) + 32 * gp;
            ds_reads[h2] = C::K_BYTES + tile_of_wave * C::DS_HALF + key_half * 4096 + n * 1024 + 16 * slot +
                           8 * ((s % 4) / 2);
        }
    }

    request_step(0, 0);
    request_step(1, 1);   // steps >= 2 always
    for (int step = 0; step < steps; ++step) {
        // this wave's share of step `step` has landed; the request of step + 1 may stay in flight
        if (step + 1 < steps) {
            wait_vector_memory<STEP_LOADS>();
        } else {
            wait_vector_memory<0>();
        }
        workgroup_barrier();
        if (step + 2 < steps) {
            request_step(step + 2, (step + 2) % 3);
        }
        const unsigned stage_offset = (step % 3) * C::STAGE_BYTES;
        unsigned k_at[2][SEL], ds_at[2];
        rebase(k_at, k_reads, stage_offset);
        rebase(ds_at, ds_reads, stage_offset);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {   // the wave's two 16-key steps
            bf16x8 ds[2];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                const int constant = qb * 2048 + kk * 256;
                const s16x4 low =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(lds + ds_at[0] + constant));
                const s16x4 high =
                    __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(lds + ds_at[1] + constant));
                ds[qb] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
            }
#pragma unroll
            for (int d = 0; d < C::D_BLOCKS; ++d) {
                const int constant = 16 * kk * C::K_ROW + (d / SEL) * (TR * 64);
                const s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (transposing_read_pointer)(lds + k_at[0][d % SEL] + constant));
                const s16x4 high = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (transposing_read_pointer)(lds + k_at[1][d % SEL] + constant));
                const bf16x8 kt =
                    __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
                dq_acc[d][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kt, ds[0], dq_acc[d][0], 0, 0, 0);
                dq_acc[d][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kt, ds[1], dq_acc[d][1], 0, 0, 0);
            }
        }
    }

    // ---- the upper key half hands its sums to the lower one: register r of lane l at
    // float (r * 64 + l) of the wave pair's area
    __syncthreads();
    {
        float* area = reinterpret_cast<float*>(lds) + (wave % 4) * (C::D_BLOCKS * 2 * 16 * 64) + lane;
        if (key_half == 1) {
#pragma unroll
            for (int d = 0; d < C::D_BLOCKS; ++d) {
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) area[((d * 2 + qb) * 16 + i) * 64] = dq_acc[d][qb][i];
                }
            }
        }
        __syncthreads();
        if (key_half == 0) {
#pragma unroll
            for (int d = 0; d < C::D_BLOCKS; ++d) {
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) dq_acc[d][qb][i] += area[((d * 2 + qb) * 16 + i) * 64];
                }
            }
        }
    }

    // ---- epilogue.  A lane holds query lq and columns 32*block + 8*(i/4) + 4*g + i%4 of its wave's column
    // blocks: stored from there, every instruction would touch 32 rows with 8 bytes each.  The rows are put
    // together in LDS instead (both column halves of a query tile side by side) and leave as whole rows,
    // 24 lanes of 16 bytes per row.
    __syncthreads();   // every wave has taken its sums out of the area the rows are staged in
    constexpr int ROW_PITCH = 2 * DQK + 16;
    if (key_half == 0) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            unsigned char* row = lds + (size_t)(tile_of_wave * QTILE + 32 * qb + lq) * ROW_PITCH;
#pragma unroll
            for (int d = 0; d < C::D_BLOCKS; ++d) {
                const int column0 = 32 * (2 * d + column_half);
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    u32x2 packed;
                    packed.x = pack_bf16(dq_acc[d][qb][4 * i4 + 0] * scale, dq_acc[d][qb][4 * i4 + 1] * scale);
                    packed.y = pack_bf16(dq_acc[d][qb][4 * i4 + 2] * scale, dq_acc[d][qb][4 * i4 + 3] * scale);
                    *reinterpret_cast<u32x2*>(row + 2 * (column0 + 8 * i4 + 4 * g)) = packed;
                }
            }
        }
    }
    __syncthreads();
    {
        constexpr int ROW_CHUNKS = DQK / 8;                      // 16-byte pieces of a row
        constexpr int PIECES = 2 * QTILE * ROW_CHUNKS;           // of the workgroup's two query tiles
        bf16_t* dq_base = query_gradient + ((size_t)b * S * heads + h) * DQK;
        const size_t q_stride = (size_t)heads * DQK;
#pragma unroll
        for (int piece = tid; piece < PIECES; piece += DQ_THREADS) {
            const int r = piece / ROW_CHUNKS;                    // row of the staged 128
            const int chunk = piece % ROW_CHUNKS;
            const int q_row = 2 * jb * QTILE + r;
            if (q_row < S) {
                const u32x4 bits = *reinterpret_cast<const u32x4*>(lds + (size_t)r * ROW_PITCH + 16 * chunk);
                *reinterpret_cast<u32x4*>(dq_base + (size_t)q_row * q_stride + 8 * chunk) = bits;
            }
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

// The dS blocks of one (batch, head) pair take about S * S bytes, so a long sequence with many heads would ask for
// tens of gigabytes if every pair kept its own.  The two gradient passes therefore run over the pairs in chunks that
// share one set of dS blocks of at most DS_BUDGET_BYTES (the chunk of a launch is a multiple of 8 pairs when it can
// be: one pair at a time per XCD); the statistics, small, are computed for all pairs at once.
// attention_backward_set_workspace_limit replaces the budget for the whole process: for callers who would rather
// trade launches for memory (and for tests of the chunked path at small sizes).
constexpr long long DS_BUDGET_BYTES = 3LL << 30;

std::atomic<long long> ds_budget_override{0};

long long ds_budget_bytes() {
    const long long value = ds_budget_override.load(std::memory_order_relaxed);
    return value > 0 ? value : DS_BUDGET_BYTES;
}

struct BackwardShape {
    int key_blocks;
    int query_tiles;
    int query_blocks;
    int sharing;                   // query heads per key/value head
    long long pairs;               // batch * key/value heads: what the launches are cut by
    long long pairs_per_launch;
    long long statistics_floats;   // every (batch, query head)
    long long ds_floats;           // one chunk of pairs, `sharing` query heads each
};

BackwardShape backward_shape(int batch_size, int sequence_length, int heads, int kv_heads) {
    BackwardShape shape;
    shape.key_blocks = (sequence_length + KBLOCK - 1) / KBLOCK;
    shape.query_tiles = (sequence_length + QTILE - 1) / QTILE;
    shape.query_blocks = shape.key_blocks;   // 128 queries per workgroup of the dQ pass
    shape.sharing = heads / kv_heads;
    shape.pairs = (long long)batch_size * kv_heads;
    shape.statistics_floats = (long long)batch_size * heads * shape.query_tiles * STAT_FLOATS;
    const long long pair_bytes = (long long)shape.sharing * ds_block_count(shape.key_blocks, shape.query_tiles) * DS_BLOCK_BYTES;
    long long chunk = pair_bytes > 0 ? ds_budget_bytes() / pair_bytes : shape.pairs;
    if (chunk >= 8) chunk -= chunk % 8;
    if (chunk < 1) chunk = 1;
    shape.pairs_per_launch = chunk < shape.pairs ? chunk : shape.pairs;
    shape.ds_floats = shape.pairs_per_launch * shape.sharing * ds_block_count(shape.key_blocks, shape.query_tiles) * DS_BLOCK_FLOATS;
    return shape;
}

template <int DQK, int DV>
void launch_backward(bf16_t* query_gradient, bf16_t* key_gradient, bf16_t* value_gradient,
                     const bf16_t* output_gradient, const bf16_t* output, const float* logsumexp,
                     const bf16_t* query, const bf16_t* key, const bf16_t* value, float* workspace, int batch_size,
                     int sequence_length, int heads, int kv_heads, float scale, hipStream_t stream) {
    using KC = KeyValueGradConfig<DQK, DV>;
    using QC = QueryGradConfig<DQK>;
    const BackwardShape shape = backward_shape(batch_size, sequence_length, heads, kv_heads);
    const long long groups = (long long)batch_size * heads;
    const long long padded_rows = groups * shape.query_tiles * QTILE;
    if ((padded_rows + 15) / 16 > 0x7fffffffLL || groups * shape.key_blocks > 0x7fffffffLL) {
        throw std::invalid_argument("attention backward: problem exceeds the grid limit");
    }
    // per-lane byte offsets inside a tile are 32-bit
    if ((long long)heads * (DQK > DV ? DQK : DV) * 2 * QTILE > 0x7fffffffLL) {
        throw std::invalid_argument("attention backward: heads * head size is too large");
    }
    float* statistics = workspace;
    unsigned char* ds_blocks = reinterpret_cast<unsigned char*>(workspace + shape.statistics_floats);
    static hip_common::OncePerDevice prepared;
    prepared.run([] {
        raise_lds_limit(attention_key_value_gradient_kernel<DQK, DV>, KC::LDS_BYTES);
        raise_lds_limit(attention_query_gradient_kernel<DQK>, QC::LDS_BYTES);
    });
    hipLaunchKernelGGL((attention_backward_statistics_kernel<DV>), dim3((unsigned)((padded_rows + 15) / 16)), dim3(256),
                       0, stream, statistics, output_gradient, output, logsumexp, batch_size, sequence_length, heads,
                       shape.query_tiles);
    HIP_CHECK(hipGetLastError());
    for (long long first = 0; first < shape.pairs; first += shape.pairs_per_launch) {
        const long long count = std::min(shape.pairs_per_launch, shape.pairs - first);
        hipLaunchKernelGGL((attention_key_value_gradient_kernel<DQK, DV>), dim3((unsigned)(count * shape.key_blocks)),
                           dim3(KV_THREADS), KC::LDS_BYTES, stream, key_gradient, value_gradient, ds_blocks, statistics,
                           output_gradient, query, key, value, sequence_length, heads, kv_heads, shape.key_blocks,
                           shape.query_tiles, (int)first, scale);
        HIP_CHECK(hipGetLastError());
        // the next chunk's first pass overwrites the dS blocks: it follows this pass in the stream.  The query
        // heads of the chunk's pairs are consecutive: count * sharing of them from first * sharing on.
        hipLaunchKernelGGL((attention_query_gradient_kernel<DQK>),
                           dim3((unsigned)(count * shape.sharing * shape.query_blocks)), dim3(DQ_THREADS), QC::LDS_BYTES,
                           stream, query_gradient, ds_blocks, key, sequence_length, heads, kv_heads, shape.query_blocks,
                           shape.key_blocks, shape.query_tiles, (int)(first * shape.sharing), scale);
        HIP_CHECK(hipGetLastError());
    }
}

}  // namespace

void attention_backward_set_workspace_limit(std::size_t bytes) {
    ds_budget_override.store(bytes > (std::size_t)1 << 62 ? 1LL << 62 : (long long)bytes, std::memory_order_relaxed);
}

std::size_t attention_backward_workspace_elements(int batch_size, int sequence_length, int heads, int kv_heads) {
    if (kv_heads <= 0 || heads % kv_heads != 0) {
        throw std::invalid_argument("attention backward: query heads must be a positive multiple of key/value heads");
    }
    const BackwardShape shape = backward_shape(batch_size, sequence_length, heads, kv_heads);
    return static_cast<std::size_t>(shape.statistics_floats + shape.ds_floats);
}

void attention_backward_dispatch(bf16_t* query_gradient, bf16_t* key_gradient, bf16_t* value_gradient,
                                 const bf16_t* output_gradient, const bf16_t* output, const float* logsumexp,
                                 const bf16_t* query, const bf16_t* key, const bf16_t* value, float* workspace,
                                 int batch_size, int sequence_length, int heads, int kv_heads, int qk_head_size,
                                 int v_head_size, float scale, hipStream_t stream) {
    if (kv_heads <= 0 || heads % kv_heads != 0) {
        throw std::invalid_argument("attention backward: query heads must be a positive multiple of key/value heads");
    }
#define DSCUDA_BWD_CASE(DQK, DV)                                                                                   \
    if (qk_head_size == DQK && v_head_size == DV) {                                                                \
        launch_backward<DQK, DV>(query_gradient, key_gradient, value_gradient, output_gradient, output, logsumexp, \
                                 query, key, value, workspace, batch_size, sequence_length, heads, kv_heads, scale, \
                                 stream);                                                                          \
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
