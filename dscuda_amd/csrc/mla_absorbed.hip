// Absorbed-query MLA backward for gfx950 (C = 512 latent + R = 64 rope, one
// shared KV head).  Takes the place of the reference's
// mla_query_backward_kernel and mla_kv_backward_kernel
// (kernels/attention/mla/sm89.cu:295-411) and keeps their contract: the four
// gradients are overwritten, the result does not depend on timing (no atomics:
// every sum has a fixed order), the caller passes no workspace.  The
// mathematics is reference/python/mla.py:42-57:
//     P = exp(S - LSE),  dP = dO latent^T,  delta = sum(dO * O),
//     dS = P (dP - delta) scale,
//     dQ = dS [latent|rope],  d[latent|rope] = dS^T [q_lat|q_rope],  dlatent += P^T dO.
//
// "Rows" are the (token, head) pairs of one batch element in memory order
// (row = token*H + head), which makes query / dO / O rows contiguous 512- and
// 64-wide vectors.  Every product runs on bf16 MFMA 32x32x16 with fp32
// accumulation on operands kept in LDS, 32 rows or keys at a time, each tile
// stored row-major once: where its row index is the contraction index the
// fragments come through transposing reads.  While a tile is multiplied the
// next one moves from registers into a second LDS buffer and the one after
// that is on its way from memory.
//
// Four launches, in this order (the order matters: the first three use the
// query-gradient buffers, which the last one overwrites, as scratch memory):
//   row statistics    delta of every row, kept in the first four bytes of the row's
//                     own 128 bytes of the rope query gradient.
//   key gradients     one shared KV head means every key is seen by all H heads of
//                     every later token: T/32 key blocks would be far too few
//                     workgroups with far too unequal work.  The (key block, row
//                     tile) visits form one list, cut into equal ranges, one per
//                     compute unit (index_math.h); a workgroup holds the keys of a
//                     block in registers and walks its row tiles: every wave forms one
//                     quadrant of S and dP of the tile, the quadrants of P and dS meet
//                     in LDS, and every wave accumulates its own four latent column
//                     blocks (key path and value path in the same accumulator) plus
//                     a rope column block.  A range that holds all visits of a key
//                     block writes the gradients, otherwise an fp32 partial result
//                     into the latent query gradient buffer.
//   reduction         sums the partial results of each cut key block in range order.
//   query gradients   a workgroup owns 32 rows and walks the keys up to the last
//                     token of those rows.  Every wave forms one quadrant of S^T and
//                     dP^T of the tile, the quadrants of dS^T meet in LDS, and every
//                     wave accumulates dQ^T for its own share of the 18 column blocks.
#include "attn_kernels.h"
#include "hip_common.h"
#include "index_math.h"

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <stdexcept>
#include <type_traits>
#include <string>

namespace dscuda {
namespace {

constexpr int RANK = 512;
constexpr int ROPE = 64;
constexpr int WIDTH = RANK + ROPE;
constexpr int TILE = 32;
constexpr int THREADS = 256;

// A [32][D] LDS tile of bf16, row-major without padding: 16-byte chunk c of row r sits at position
// c ^ tile_swizzle(r), which spreads both the 16-byte reads down a column and the transposing reads over the banks.
template <int D>
struct Tile32 {
    static constexpr int ROW = 2 * D;
    static constexpr int BYTES = TILE * ROW;
    using Read = index_math::TileReadMath<ROW>;
    static constexpr int PARTS = Read::TR;   // per-lane address parts a fragment read chooses from
};

// One thread's share of a [32][D_PART] tile in registers: 16-byte pieces of rows.
template <int D_PART>
struct TileShare {
    static constexpr int PIECES = TILE * D_PART / 8;
    static constexpr int PER_THREAD = (PIECES + THREADS - 1) / THREADS;
    u32x4 r[PER_THREAD];
};

// Fetch a [32][D_PART] tile whose rows lie one behind the other in memory from `first`; rows from `valid_rows`
// on (possibly <= 0) are zero.
template <int D_PART>
__device__ __forceinline__ void fetch_tile(TileShare<D_PART>& share, const bf16_t* first, int valid_rows, int tid) {
    using S = TileShare<D_PART>;
#pragma unroll
    for (int p = 0; p < S::PER_THREAD; ++p) {
        const int piece = tid + p * THREADS;
        share.r[p] = u32x4{0, 0, 0, 0};
        if (piece < S::PIECES && piece / (D_PART / 8) < valid_rows) {
            share.r[p] = *reinterpret_cast<const u32x4*>(first + 8 * piece);
        }
    }
}

// Place a fetched share into columns [column0, column0 + D_PART) of a [32][D] LDS tile, so that a tile can be
// assembled from two tensors.
template <int D, int D_PART>
__device__ __forceinline__ void place_tile(const TileShare<D_PART>& share, unsigned char* tile, int column0, int tid) {
    using S = TileShare<D_PART>;
#pragma unroll
    for (int p = 0; p < S::PER_THREAD; ++p) {
        const int piece = tid + p * THREADS;
        if (piece >= S::PIECES) break;
        const int row = piece / (D_PART / 8);
        const int chunk = column0 / 8 + piece % (D_PART / 8);
        *reinterpret_cast<u32x4*>(tile + row * Tile32<D>::ROW +
                                  16 * (chunk ^ index_math::tile_swizzle<Tile32<D>::ROW>(row))) = share.r[p];
    }
}

// Operand with the tile's row as the contraction index, through transposing reads (ds_read_b64_tr_b16): in a
// block of 16 lanes, lane s points at row 4*g + s/4 (+8 for the second read), columns 4*(s%4)..+3 of the block's
// 16 columns, and receives the four rows' values of column s.  The lane ends up with column lane%32 of a
// 32-column block and tile rows {16n + 4g .. +3, 16n + 8 + 4g .. +3}, the order in which the accumulators of the
// score products hold rows.  `low` / `high`: the lane's addresses of the two reads inside the tile's first 16
// rows (TransposedAt), `offset` what is the same for all lanes.
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4* transposing_read_pointer;

__device__ __forceinline__ bf16x8 transposed_fragment(const unsigned char* tile, int low_at, int high_at, int offset) {
    const s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(tile + low_at + offset));
    const s16x4 high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(tile + high_at + offset));
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
}

// The lane's addresses for column block b: part b % PARTS, plus (b / PARTS) * 64 * PARTS bytes.
template <int D>
struct TransposedAt {
    int low[Tile32<D>::PARTS], high[Tile32<D>::PARTS];
    __device__ __forceinline__ TransposedAt(int lane, int extra_bytes) {
#pragma unroll
        for (int i = 0; i < Tile32<D>::PARTS; ++i) {
            low[i] = (int)Tile32<D>::Read::transposed(0, i, lane) + extra_bytes;
            high[i] = (int)Tile32<D>::Read::transposed(1, i, lane) + extra_bytes;
        }
    }
};

__device__ __forceinline__ void clear(f32x16& value) {
#pragma unroll
    for (int i = 0; i < 16; ++i) value[i] = 0.f;
}

// f(integral_constant<int, BEGIN>) ... f(integral_constant<int, END - 1>)
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// COUNT MFMAs, each fed by one LDS fragment read AHEAD steps before its use: with one wave per SIMD nothing
// else hides the latency of the reads.  `ring` holds fragments 0 .. AHEAD-1 on entry.
template <int COUNT, int AHEAD, typename Fragment, typename Multiply>
__device__ __forceinline__ void fragment_stream(bf16x8 (&ring)[AHEAD], Fragment&& fragment, Multiply&& multiply) {
    static_for<0, COUNT>([&](auto tag) {
        constexpr int I = decltype(tag)::value;
        multiply(tag, ring[I % AHEAD]);
        if constexpr (I + AHEAD < COUNT) ring[I % AHEAD] = fragment(std::integral_constant<int, I + AHEAD>{});
        __builtin_amdgcn_sched_barrier(0);
    });
}

template <int AHEAD, typename Fragment>
__device__ __forceinline__ void fill_ring(bf16x8 (&ring)[AHEAD], Fragment&& fragment) {
    static_for<0, AHEAD>([&](auto tag) { ring[decltype(tag)::value] = fragment(tag); });
}

// The score products of a 32 x 32 tile are split over the four waves: each forms one 16 x 16 quadrant (16x16x32
// MFMA: lane l holds column l%16 and rows 4*(l/16) .. +3 of its quadrant), applies the softmax gradient to it and
// leaves its P / dS values in an LDS tile [32 columns][32 rows] of bf16, from which every wave reads the whole
// tile as an operand of the 32x32x16 products: lane l takes column l%32, rows {16n + 4g .. +3, 16n + 8 + 4g .. +3}
// (g = l/32), the row order of the transposing reads that feed the other operand.  72-byte pitch: the 8-byte
// accesses of 32 lanes fall into different banks.
constexpr int EXCHANGE_PITCH = 2 * TILE + 8;
constexpr int EXCHANGE_BYTES = TILE * EXCHANGE_PITCH;

// four neighbouring rows (from `row`, a multiple of 4) of column `column`
__device__ __forceinline__ void exchange_store(unsigned char* exchange, int column, int row, const float (&value)[4]) {
    u32x2 packed;
    packed.x = pack_bf16(value[0], value[1]);
    packed.y = pack_bf16(value[2], value[3]);
    *reinterpret_cast<u32x2*>(exchange + column * EXCHANGE_PITCH + 2 * row) = packed;
}

__device__ __forceinline__ bf16x8 exchange_fragment(const unsigned char* exchange, int lq, int g, int n) {
    const unsigned char* at = exchange + lq * EXCHANGE_PITCH + 2 * (16 * n + 4 * g);
    const u32x2 low = *reinterpret_cast<const u32x2*>(at);
    const u32x2 high = *reinterpret_cast<const u32x2*>(at + 16);
    return __builtin_bit_cast(bf16x8, u32x4{low.x, low.y, high.x, high.y});
}

// Operand of the 16x16x32 products out of a tile: row 16*half + lane%16, k-step s of 32 columns: part s % PARTS
// of the lane's addresses, plus (s / PARTS) * 64 * PARTS bytes.
template <int D>
struct QuadrantAt {
    int at[Tile32<D>::PARTS];
    __device__ __forceinline__ QuadrantAt(int lane, int half) {
#pragma unroll
        for (int i = 0; i < Tile32<D>::PARTS; ++i) {
            at[i] = (int)Tile32<D>::Read::quadrant(i, lane) + half * 16 * Tile32<D>::ROW;
        }
    }
};

template <int S, int D>
__device__ __forceinline__ bf16x8 quadrant_fragment(const unsigned char* tile, const QuadrantAt<D>& lane_at) {
    constexpr int PARTS = Tile32<D>::PARTS;
    return *reinterpret_cast<const bf16x8*>(tile + lane_at.at[S % PARTS] + (S / PARTS) * 64 * PARTS);
}

// The same operand straight from memory: 32 columns per step, latent part first, then the rope part.
template <int STEPS>
__device__ __forceinline__ void fetch_quadrant_operand(bf16x8 (&operand)[STEPS], const bf16_t* latent_row,
                                                       const bf16_t* rope_row, bool valid, int quad) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        u32x4 bits = {0, 0, 0, 0};
        if (valid) {
            const bf16_t* source = s < RANK / 32 ? latent_row + 32 * s + 8 * quad : rope_row + 32 * (s - RANK / 32) + 8 * quad;
            bits = *reinterpret_cast<const u32x4*>(source);
        }
        operand[s] = __builtin_bit_cast(bf16x8, bits);
    }
}

// delta = sum(dO * O) of a row is kept in the first four bytes of the row's 64 rope query gradients (which the
// query-gradient kernel, the last of the call, overwrites after it has read the delta of its own rows).
constexpr int DELTA_STRIDE = ROPE / 2;   // in floats

// Eight threads share a row: thread `part` takes the 16 bytes at 16 * part of each of the row's eight 128-byte
// pieces, so that an instruction of the eight reads 128 bytes in a row; rows of all batch elements are numbered through.
__global__ __launch_bounds__(THREADS) void mla_absorbed_row_statistics_kernel(
    float* delta, const bf16_t* __restrict__ output_gradient, const bf16_t* __restrict__ output, long long rows) {
    const int tid = threadIdx.x;
    const int part = tid % 8;
    const long long row = (long long)blockIdx.x * TILE + tid / 8;
    float sum = 0.f;
    if (row < rows) {
        const bf16_t* a_row = output_gradient + row * RANK + 8 * part;
        const bf16_t* b_row = output + row * RANK + 8 * part;
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(a_row + 64 * v);
            const u32x4 b = *reinterpret_cast<const u32x4*>(b_row + 64 * v);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sum += bf16_bits_to_float(a[j] & 0xffffu) * bf16_bits_to_float(b[j] & 0xffffu);
                sum += bf16_bits_to_float(a[j] >> 16) * bf16_bits_to_float(b[j] >> 16);
            }
        }
    }
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    sum += __shfl_xor(sum, 4);
    if (part == 0 && row < rows) delta[row * DELTA_STRIDE] = sum;
}

// What the gradient formulas need of one row besides its vectors.
struct RowStatistics {
    float lse;     // as loaded: whoever multiplies it (by log2(e)) waits for the load, so that is left to the user
    float delta;
    int token;     // -1: no such row, it sees no key
};

// Row `row` of the batch element whose rows start at `batch_row0` (thread-per-row: the first 32 threads of a tile).
__device__ __forceinline__ RowStatistics fetch_row_statistics(const float* delta, const float* lse_batch,
                                                              long long batch_row0, long long row, long long rows,
                                                              int heads, int sequence_length) {
    RowStatistics statistics = {0.f, 0.f, -1};
    if (row < rows) {
        const int token = (int)(row / heads);
        const int head = (int)(row % heads);
        statistics.lse = lse_batch[(size_t)head * sequence_length + token];
        statistics.delta = delta[(batch_row0 + row) * DELTA_STRIDE];
        statistics.token = token;
    }
    return statistics;
}

// ---- query gradients -----------------------------------------------------------

constexpr int QUERY_THREADS = 512;
constexpr int QUERY_ROWS = 64;   // rows of one workgroup: every key tile it fetches serves two row tiles

struct QueryGradLayout {
    static constexpr int K_LATENT = 0;                                    // [32 keys][512]
    static constexpr int K_ROPE = K_LATENT + Tile32<RANK>::BYTES;         // [32 keys][64]
    static constexpr int BUFFER_BYTES = K_ROPE + Tile32<ROPE>::BYTES;
    static constexpr int EXCHANGE = 2 * BUFFER_BYTES;                     // the tile in use and the one arriving
    static constexpr int EXCHANGE_PAIR = 2 * EXCHANGE_BYTES;              // dS of the two row tiles against one key tile
    static constexpr int LDS_BYTES = EXCHANGE + 2 * EXCHANGE_PAIR;        // of the key tile being scored and the one before
};

// Eight waves, two per SIMD, in two roles (the design of the key-gradient kernel below, turned round: here the rows
// stay and the key tiles pass).  Waves 0..3 form the scores: wave w holds rows 16*w .. +15 of the workgroup's 64
// as register operands (query and dO row), multiplies every key fragment it reads from LDS into the score and the
// dP product, applies the softmax gradient and leaves dS in the exchange tile of its row tile.  Waves 4..7 hold
// the sums: wave 4 + v the latent column blocks 4*v .. +3 of BOTH row tiles (a key fragment read once serves two
// products) and rope block v % 2 of row tile v / 2; they keep the transposed fragments of the key tile BEFORE in
// registers, multiply them with that tile's dS while the next scores are formed, and replace each by the same
// fragment of the tile being scored.  So one key tile is read at
// a time, the other buffer is free during the whole step and the next tile goes straight from memory into it
// (global_load_lds, requested from inside the product streams, awaited before the step's one barrier).  Each SIMD
// carries a score wave (68 products of 16x16x32) and a gradient wave (18 of 32x32x16).
// The walk is compiled once per role so that the roles share the register file.
template <bool SCORES>
__device__ __forceinline__ void query_gradient_walk(
    bf16_t* query_latent_gradient, bf16_t* query_rope_gradient, const float* delta_of_rows,
    const bf16_t* __restrict__ output_gradient, const float* __restrict__ logsumexp,
    const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int sequence_length, int heads,
    int row_blocks, float scale) {
    using L = QueryGradLayout;
    using Wide = Tile32<RANK>;
    using Narrow = Tile32<ROPE>;
    constexpr int Q_STEPS = WIDTH / 32;   // 18
    constexpr int O_STEPS = RANK / 32;    // 16
    constexpr int AHEAD = 6;
    constexpr int LATENT_BLOCKS = 4;      // per gradient wave, of each row tile
    constexpr int HELD = LATENT_BLOCKS + 1;   // fragments per 16-key step: the latent blocks and the rope block
    constexpr int ROWS_PER_WAVE = TILE / 8;   // key rows of the wide tile a wave requests

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    __builtin_assume(tid >= 0 && tid < QUERY_THREADS);
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int l16 = lane % 16;
    const int quad = lane / 16;
    const int T = sequence_length;

    const int batch = blockIdx.x / row_blocks;
    const int row_block = row_blocks - 1 - blockIdx.x % row_blocks;   // latest rows (most keys) first
    const long long rows = (long long)T * heads;
    const long long row0 = (long long)row_block * QUERY_ROWS;
    const long long batch_row0 = (long long)batch * rows;
    const bf16_t* latent = kv_latent + (size_t)batch * T * RANK;
    const bf16_t* rope = key_rope + (size_t)batch * T * ROPE;

    const long long last_row = min(rows, row0 + QUERY_ROWS) - 1;
    const int visible = (int)(last_row / heads) + 1;
    const int tiles = (visible + TILE - 1) / TILE;
    const float c = scale * LOG2E;

    // Requests of a key tile: the wave brings key rows 4*wave .. +3 of the wide tile (an instruction fills one row:
    // lane l fetches the chunk that belongs at position l), waves 0..3 also instruction `wave` of the narrow tile
    // (eight rows of eight chunks).  Keys past the last one repeat it: every row's token is below them, so their
    // dS is zero whatever they hold.
    const unsigned lds_base = lds_offset_of(lds);
    unsigned wide_part[ROWS_PER_WAVE];
#pragma unroll
    for (int j = 0; j < ROWS_PER_WAVE; ++j) {
        wide_part[j] = 16u * (unsigned)(lane ^ index_math::tile_swizzle<Wide::ROW>(ROWS_PER_WAVE * wave + j));
    }
    const int narrow_row = 8 * (wave % 4) + lane / 8;
    const unsigned narrow_part = 16u * (unsigned)((lane % 8) ^ index_math::tile_swizzle<Narrow::ROW>(narrow_row));
    constexpr int REQUESTS = ROWS_PER_WAVE + 1;
    struct {
        const bf16_t* latent;
        const bf16_t* rope;
        int last_valid;
        unsigned buffer;
    } arriving;
    auto begin_requests = [&](int tile, int parity) {
        const int key0 = tile * TILE;
        arriving.latent = latent + (size_t)key0 * RANK;
        arriving.rope = rope + (size_t)key0 * ROPE;
        arriving.last_valid = min(T - key0, TILE) - 1;
        arriving.buffer = lds_base + parity * L::BUFFER_BYTES;
    };
    auto request = [&](auto tag) {
        constexpr int R = decltype(tag)::value;
        if constexpr (R < ROWS_PER_WAVE) {
            const int row = ROWS_PER_WAVE * wave + R;
            direct_load_16_offset(arriving.latent, wide_part[R] + (unsigned)(min(row, arriving.last_valid) * Wide::ROW),
                                  arriving.buffer + L::K_LATENT + row * Wide::ROW);
        } else if constexpr (R == ROWS_PER_WAVE) {
            if constexpr (SCORES) {
                direct_load_16_offset(arriving.rope, narrow_part + (unsigned)(min(narrow_row, arriving.last_valid) * Narrow::ROW),
                                      arriving.buffer + L::K_ROPE + 8 * wave * Narrow::ROW);
            }
        }
    };

    // score waves: rows 16*wave .. +15 as B operands (column = row l16): the query row and its dO row
    bf16x8 qf[Q_STEPS], dof[O_STEPS];
    float row_lse2 = 0.f, row_delta = 0.f;
    int row_token = -1;
    const QuadrantAt<RANK> wide_quadrant(lane, 0);
    const QuadrantAt<ROPE> narrow_quadrant(lane, 0);
    if constexpr (SCORES) {
        const long long own_row = row0 + 16 * wave + l16;
        const bool own_valid = own_row < rows;
        const size_t own = batch_row0 + (own_valid ? own_row : 0);
        fetch_quadrant_operand(qf, query_latent + own * RANK, query_rope + own * ROPE, own_valid, quad);
        fetch_quadrant_operand(dof, output_gradient + own * RANK, nullptr, own_valid, quad);
        const RowStatistics statistics = fetch_row_statistics(delta_of_rows, logsumexp + (size_t)batch * heads * T,
                                                              batch_row0, own_row, rows, heads, T);
        row_lse2 = statistics.lse * LOG2E;
        row_delta = statistics.delta;
        row_token = statistics.token;
    }

    // gradient waves: latent column blocks 4*v .. +3 of both row tiles, rope block v % 2 of row tile v / 2
    const int v = wave % 4;
    const int rope_tile = v / 2;
    const int rope_block = v % 2;
    const TransposedAt<RANK> wide_columns(lane, 256 * v);
    const int rope_columns_low = (int)Narrow::Read::transposed(0, rope_block, lane);
    const int rope_columns_high = (int)Narrow::Read::transposed(1, rope_block, lane);
    f32x16 dq_acc[2][LATENT_BLOCKS], rope_acc;
    bf16x8 held[2 * HELD];   // the column fragments of the key tile before the one in LDS (zero before the first)
    if constexpr (!SCORES) {
#pragma unroll
        for (int j = 0; j < LATENT_BLOCKS; ++j) {
            clear(dq_acc[0][j]);
            clear(dq_acc[1][j]);
        }
        clear(rope_acc);
#pragma unroll
        for (int f = 0; f < 2 * HELD; ++f) held[f] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
    }

    // (keys x rows) quadrants of 16 x 16, lane holds row l16 and keys 4*quad .. +3 of each key half.  A key fragment
    // of the latent part serves the score product and the dP product.
    auto score_tile = [&](const unsigned char* buffer, unsigned char* exchange, int key0) {
        const unsigned char* k_latent = buffer + L::K_LATENT;
        const unsigned char* k_rope = buffer + L::K_ROPE;
        f32x4 s_acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        f32x4 dp_acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        bf16x8 ring[AHEAD];
        auto key_fragment = [&](auto tag) {
            constexpr int S = decltype(tag)::value / 2;
            constexpr int KH = decltype(tag)::value % 2;
            if constexpr (S < O_STEPS) {
                return quadrant_fragment<S>(k_latent + KH * 16 * Wide::ROW, wide_quadrant);
            } else {
                return quadrant_fragment<S - O_STEPS>(k_rope + KH * 16 * Narrow::ROW, narrow_quadrant);
            }
        };
        fill_ring(ring, key_fragment);
        fragment_stream<2 * Q_STEPS>(ring, key_fragment, [&](auto tag, const bf16x8& fragment) {
            constexpr int I = decltype(tag)::value;
            constexpr int S = I / 2;
            constexpr int KH = I % 2;
            s_acc[KH] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, qf[S], s_acc[KH], 0, 0, 0);
            if constexpr (S < O_STEPS) {
                dp_acc[KH] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, dof[S], dp_acc[KH], 0, 0, 0);
            }
            if constexpr (I % 7 == 0) request(std::integral_constant<int, I / 7>{});
        });
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
            float ds[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int k = key0 + 16 * kh + 4 * quad + i;
                float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[kh][i], c, -row_lse2));
                if (k > row_token) probability = 0.f;
                ds[i] = probability * (dp_acc[kh][i] - row_delta) * scale;
            }
            exchange_store(exchange, 16 * (wave % 2) + l16, 16 * kh + 4 * quad, ds);   // [row][key]
        }
    };

    // dQ^T += K^T dS^T: the held fragments (key tile t - 1) meet dS of that tile (of both row tiles), and each
    // gives way to the same fragment of tile t in `buffer`
    auto add_tile = [&](const unsigned char* buffer, const unsigned char* exchange, bool any) {
        const unsigned char* k_latent = buffer + L::K_LATENT;
        const unsigned char* k_rope = buffer + L::K_ROPE;
        bf16x8 dsf[2][2];   // [row tile][16-key step]
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                dsf[t][n] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
                if (any) dsf[t][n] = exchange_fragment(exchange + t * EXCHANGE_BYTES, lq, g, n);
            }
        }
        static_for<0, 2 * HELD>([&](auto tag) {
            constexpr int I = decltype(tag)::value;
            constexpr int N = I / HELD;
            constexpr int F = I % HELD;
            if constexpr (F < LATENT_BLOCKS) {
                dq_acc[0][F] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(held[I], dsf[0][N], dq_acc[0][F], 0, 0, 0);
                dq_acc[1][F] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(held[I], dsf[1][N], dq_acc[1][F], 0, 0, 0);
                held[I] = transposed_fragment(k_latent, wide_columns.low[F], wide_columns.high[F], N * 16 * Wide::ROW);
            } else {
                const bf16x8 own = rope_tile == 0 ? dsf[0][N] : dsf[1][N];
                rope_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(held[I], own, rope_acc, 0, 0, 0);
                held[I] = transposed_fragment(k_rope, rope_columns_low, rope_columns_high, N * 16 * Narrow::ROW);
            }
            if constexpr (I % 2 == 0) request(std::integral_constant<int, I / 2>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // Step t: key tile t is in buffer t % 2 (scored there, and picked up by the gradient waves for step t + 1), tile
    // t + 1 arrives in the other buffer; past the last tile the last one is requested again, into a buffer nobody
    // reads, which keeps the streams free of branches.  One more step lets the gradient waves catch up.
    begin_requests(0, 0);
    static_for<0, REQUESTS>(request);
    wait_vector_memory<0>();
    workgroup_barrier();
    for (int tile = 0; tile <= tiles; ++tile) {
        const int parity = tile & 1;
        begin_requests(tile + 1 < tiles ? tile + 1 : tiles - 1, parity ^ 1);
        if constexpr (SCORES) {
            if (tile < tiles) {
                score_tile(lds + parity * L::BUFFER_BYTES,
                           lds + L::EXCHANGE + parity * L::EXCHANGE_PAIR + (wave / 2) * EXCHANGE_BYTES, tile * TILE);
            }
        } else {
            add_tile(lds + parity * L::BUFFER_BYTES, lds + L::EXCHANGE + (parity ^ 1) * L::EXCHANGE_PAIR, tile > 0);
        }
        wait_vector_memory<0>();
        workgroup_barrier();   // tile t has been read, its dS and tile t + 1 are in place
    }

    // gradient waves: lane holds row lq of a row tile and columns 32*block + 8*(i/4) + 4*g + i%4
    if constexpr (!SCORES) {
        auto store_block = [&](const f32x16& sums, long long row, bf16_t* gradient, int width, int column0) {
            if (row < rows) {
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    u32x2 packed;
                    packed.x = pack_bf16(sums[4 * i4 + 0], sums[4 * i4 + 1]);
                    packed.y = pack_bf16(sums[4 * i4 + 2], sums[4 * i4 + 3]);
                    *reinterpret_cast<u32x2*>(gradient + (batch_row0 + row) * width + column0 + 8 * i4 + 4 * g) = packed;
                }
            }
        };
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int j = 0; j < LATENT_BLOCKS; ++j) {
                store_block(dq_acc[t][j], row0 + TILE * t + lq, query_latent_gradient, RANK, 32 * (LATENT_BLOCKS * v + j));
            }
        }
        store_block(rope_acc, row0 + TILE * rope_tile + lq, query_rope_gradient, ROPE, 32 * rope_block);
    }
}

__global__ __launch_bounds__(QUERY_THREADS) void mla_absorbed_query_gradient_kernel(
    bf16_t* query_latent_gradient, bf16_t* query_rope_gradient, const float* delta_of_rows,
    const bf16_t* __restrict__ output_gradient, const float* __restrict__ logsumexp,
    const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int sequence_length, int heads,
    int row_blocks, float scale) {
    if (threadIdx.x < QUERY_THREADS / 2) {
        query_gradient_walk<true>(query_latent_gradient, query_rope_gradient, delta_of_rows, output_gradient, logsumexp,
                                  query_latent, query_rope, kv_latent, key_rope, sequence_length, heads, row_blocks, scale);
    } else {
        query_gradient_walk<false>(query_latent_gradient, query_rope_gradient, delta_of_rows, output_gradient, logsumexp,
                                   query_latent, query_rope, kv_latent, key_rope, sequence_length, heads, row_blocks, scale);
    }
}

// ---- key gradients -------------------------------------------------------------

struct KeyGradLayout {
    static constexpr int Q_LATENT = 0;                                   // [32 rows][512]
    static constexpr int DO_ROWS = Q_LATENT + Tile32<RANK>::BYTES;       // [32 rows][512]
    static constexpr int Q_ROPE = DO_ROWS + Tile32<RANK>::BYTES;         // [32 rows][64]
    static constexpr int STATS = Q_ROPE + Tile32<ROPE>::BYTES;
    static constexpr int BUFFER_BYTES = STATS + 3 * TILE * 4;
    static constexpr int EXCHANGE = 2 * BUFFER_BYTES;                    // the tile in use and the one arriving
    static constexpr int EXCHANGE_PAIR = 2 * EXCHANGE_BYTES;             // P and dS of one tile
    static constexpr int LDS_BYTES = EXCHANGE + 2 * EXCHANGE_PAIR;       // of the tile being scored and the one before
};

constexpr int PARTIAL_FLOATS = TILE * WIDTH;   // one slot of partial key gradients: [32 keys][576] fp32
static_assert(PARTIAL_FLOATS * 4 == index_math::KEY_PARTIAL_BYTES, "slot size");

// `interval_length` > 0: workgroup w takes item w of the interval cut (index_math.h), slot w.  Otherwise `ranges` > 0:
// workgroup w walks range w of the list of visits; 0: workgroup w walks all visits of key block w (numbered through
// the batch elements) and writes the gradients itself.
//
// The four waves have two roles.  Waves 0 and 1 form the scores of a row tile: each takes 16 rows against all
// 32 keys (the keys as register operands, every row fragment read from LDS feeds both key halves), applies the
// softmax gradient and leaves P and dS in an exchange tile.  Waves 2 and 3 hold the gradient sums, nine column
// blocks each (eight latent, one rope), and multiply the exchange tiles of the row tile BEFORE into them while the
// next scores are formed: the two roles load the matrix pipes of their SIMDs equally (68 products of 16x16x32
// against 34 of 32x32x16) and run side by side, where one wave doing both in turn would leave its pipe idle
// during every LDS round trip.
//
// The gradient waves keep the column fragments of that earlier tile in registers: while a step's products consume
// them one by one, each is replaced by the same fragment of the tile being scored, for the next step.  So only one
// tile is read from LDS at a time, the other buffer is free for the whole step, and the rows of the next tile go
// straight from memory into it (global_load_lds, issued at the start of the step, awaited at its end): no registers,
// no LDS write instructions and no separate phase for them, and a step has one barrier.
//
// The walk is compiled once per role (SCORES), the kernel branches into one of the two: the key operands of the
// score waves and the sums and fragments of the gradient waves then share the register file.  Both roles pass the
// same barriers in the same order.
template <bool SCORES>
__device__ __forceinline__ void key_gradient_walk(
    bf16_t* __restrict__ kv_latent_gradient, bf16_t* __restrict__ key_rope_gradient, float* __restrict__ partial_slots,
    const float* __restrict__ delta_of_rows, const bf16_t* __restrict__ output_gradient,
    const float* __restrict__ logsumexp, const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int batch_size, int sequence_length,
    int heads, int ranges, int interval_length, float scale) {
    using L = KeyGradLayout;
    using Wide = Tile32<RANK>;             // the latent query rows and the dO rows
    using Narrow = Tile32<ROPE>;           // the rope query rows
    constexpr int Q_STEPS = WIDTH / 32;    // 18
    constexpr int O_STEPS = RANK / 32;     // 16
    constexpr int AHEAD = 6;
    constexpr int LATENT_BLOCKS = 8;       // per gradient wave
    constexpr int PER_STEP = 2 * LATENT_BLOCKS + 1;   // column fragments per 16-row step of a gradient wave
    constexpr int ROWS_PER_WAVE = TILE / 4;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    __builtin_assume(tid >= 0 && tid < THREADS);
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int T = sequence_length;
    const long long rows = (long long)T * heads;
    const float c = scale * LOG2E;
    const int half = wave % 2;             // score waves: rows 16*half .. +15; gradient waves: column blocks 8*half .. +7, 16 + half
    const int l16 = lane % 16;
    const int quad = lane / 16;
    const QuadrantAt<RANK> wide_quadrant(lane, half);
    const QuadrantAt<ROPE> narrow_quadrant(lane, half);
    const TransposedAt<RANK> wide_columns(lane, 512 * half);
    const int rope_columns_low = (int)Narrow::Read::transposed(0, half, lane);
    const int rope_columns_high = (int)Narrow::Read::transposed(1, half, lane);

    // Requests: the wave brings rows 8*wave .. +7 of the two wide tiles (an instruction fills one row: lane l
    // fetches the chunk that belongs at position l) and instruction `wave` of the narrow tile (eight rows of eight chunks).
    const unsigned lds_base = lds_offset_of(lds);
    unsigned wide_part[ROWS_PER_WAVE];
#pragma unroll
    for (int j = 0; j < ROWS_PER_WAVE; ++j) {
        wide_part[j] = 16u * (unsigned)(lane ^ index_math::tile_swizzle<Wide::ROW>(ROWS_PER_WAVE * wave + j));
    }
    const int narrow_row = ROWS_PER_WAVE * wave + lane / 8;
    const unsigned narrow_part = 16u * (unsigned)((lane % 8) ^ index_math::tile_swizzle<Narrow::ROW>(narrow_row));

    const index_math::KeyVisits visits = index_math::key_visits(T, heads);
    const long long per_batch = visits.per_batch();
    const long long total = per_batch * batch_size;
    long long position, range_end;
    long long item = 0;
    if (interval_length > 0) {
        const index_math::KeyIntervals cut = index_math::key_intervals(T, heads, interval_length);
        const long long items = cut.items();
        item = blockIdx.x;
        const int batch = (int)(item / items);
        int interval, key_block;
        cut.locate(item - batch * items, interval, key_block);
        const int first = max(interval * interval_length, visits.first_tile(key_block));
        position = batch * per_batch + visits.before(key_block) + (first - visits.first_tile(key_block));
        range_end = position + (cut.end_of(interval) - first);
    } else if (ranges > 0) {
        position = index_math::wide_range_begin(total, ranges, blockIdx.x);
        range_end = index_math::wide_range_begin(total, ranges, blockIdx.x + 1);
    } else {
        const int batch = blockIdx.x / visits.key_blocks;
        const int key_block = blockIdx.x % visits.key_blocks;
        position = batch * per_batch + visits.before(key_block);
        range_end = batch * per_batch + visits.before(key_block + 1);
    }

    while (position < range_end) {
        const int batch = (int)(position / per_batch);
        const long long within = position - batch * per_batch;
        const int key_block = visits.block_of(within);
        const long long block_begin = visits.before(key_block);
        const long long block_end = visits.before(key_block + 1);
        const long long segment_end = min(range_end - batch * per_batch, block_end);
        const int first_tile = visits.first_tile(key_block) + (int)(within - block_begin);
        const int end_tile = visits.first_tile(key_block) + (int)(segment_end - block_begin);
        const bool whole = within == block_begin && segment_end == block_end;

        const int k0 = key_block * TILE;
        const long long batch_row0 = (long long)batch * rows;
        const bf16_t* ql = query_latent + batch_row0 * RANK;
        const bf16_t* qr = query_rope + batch_row0 * ROPE;
        const bf16_t* dout = output_gradient + batch_row0 * RANK;
        const bf16_t* latent = kv_latent + (size_t)batch * T * RANK;
        const bf16_t* rope = key_rope + (size_t)batch * T * ROPE;
        const float* lse_batch = logsumexp + (size_t)batch * heads * T;

        // score waves: the keys as B operands (column = key 16*kh + l16); the value operand is the latent part
        bf16x8 kf[2][Q_STEPS];
        if constexpr (SCORES) {
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                const int own_key = k0 + 16 * kh + l16;
                const size_t k = own_key < T ? own_key : 0;
                fetch_quadrant_operand(kf[kh], latent + k * RANK, rope + k * ROPE, own_key < T, quad);
            }
        }

        // gradient waves: column blocks 8*half + j of the latent part, block half of the rope part; and the column
        // fragments of the tile before the one in LDS (zero before the first: its products add nothing)
        f32x16 latent_acc[LATENT_BLOCKS], rope_acc;
        bf16x8 held[2 * PER_STEP];
        if constexpr (!SCORES) {
#pragma unroll
            for (int j = 0; j < LATENT_BLOCKS; ++j) clear(latent_acc[j]);
            clear(rope_acc);
#pragma unroll
            for (int f = 0; f < 2 * PER_STEP; ++f) held[f] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
        }

        // Rows of a tile past the last row of the batch element repeat that row: their token is -1, which sees no
        // key, so their P and dS are zero whatever the rows hold.  The wave's REQUESTS requests of a tile are issued
        // one by one from inside the product streams (issued in one go they fill the queue of the memory pipe and
        // the wave stands still until it drains); past the last tile of the segment the last tile is requested again,
        // into a buffer nobody reads, which keeps the streams free of branches.
        constexpr int REQUESTS = 2 * ROWS_PER_WAVE + 1;
        struct {
            const bf16_t* latent;
            const bf16_t* gradient;
            const bf16_t* rope;
            int last_valid;
            unsigned buffer;
        } arriving;
        RowStatistics statistics = {0.f, 0.f, -1};
        auto begin_requests = [&](int tile, int parity) {
            const long long row0 = (long long)tile * TILE;
            arriving.latent = ql + row0 * RANK;
            arriving.gradient = dout + row0 * RANK;
            arriving.rope = qr + row0 * ROPE;
            arriving.last_valid = (int)min(rows - row0, (long long)TILE) - 1;
            arriving.buffer = lds_base + parity * L::BUFFER_BYTES;
            // the statistics of its rows: one lane per row, in a gradient wave (the score waves have more to do)
            if (tid >= 2 * 64 && tid < 2 * 64 + TILE) {
                const int r = tid - 2 * 64;
                statistics = {0.f, 0.f, -1};
                if (r <= arriving.last_valid) {
                    // rows fit 31 bits as a rule: 32-bit division is a fraction of the 64-bit one
                    int token, head;
                    if (rows <= 0x7fffffffLL) {
                        const unsigned row = (unsigned)row0 + (unsigned)r;
                        token = (int)(row / (unsigned)heads);
                        head = (int)(row % (unsigned)heads);
                    } else {
                        token = (int)((row0 + r) / heads);
                        head = (int)((row0 + r) % heads);
                    }
                    statistics.lse = lse_batch[(size_t)head * T + token];
                    statistics.delta = delta_of_rows[(batch_row0 + row0 + r) * DELTA_STRIDE];
                    statistics.token = token;
                }
            }
        };
        auto request = [&](auto tag) {
            constexpr int R = decltype(tag)::value;
            if constexpr (R < 2 * ROWS_PER_WAVE) {
                constexpr int J = R / 2;
                const int row = ROWS_PER_WAVE * wave + J;
                const unsigned source = wide_part[J] + (unsigned)(min(row, arriving.last_valid) * Wide::ROW);
                if constexpr (R % 2 == 0) {
                    direct_load_16_offset(arriving.latent, source, arriving.buffer + L::Q_LATENT + row * Wide::ROW);
                } else {
                    direct_load_16_offset(arriving.gradient, source, arriving.buffer + L::DO_ROWS + row * Wide::ROW);
                }
            } else if constexpr (R == 2 * ROWS_PER_WAVE) {
                direct_load_16_offset(arriving.rope, narrow_part + (unsigned)(min(narrow_row, arriving.last_valid) * Narrow::ROW),
                                      arriving.buffer + L::Q_ROPE + ROWS_PER_WAVE * wave * Narrow::ROW);
            }
        };
        // after the wave's requests have arrived
        auto place_statistics = [&](int parity) {
            if (tid >= 2 * 64 && tid < 2 * 64 + TILE) {
                const int r = tid - 2 * 64;
                float* lse2 = reinterpret_cast<float*>(lds + parity * L::BUFFER_BYTES + L::STATS);
                lse2[r] = statistics.lse * LOG2E;
                lse2[TILE + r] = statistics.delta;
                reinterpret_cast<int*>(lse2)[2 * TILE + r] = statistics.token;
            }
        };

        // scores of one tile: (rows x keys) quadrants of 16 x 16, lane holds key 16*kh + l16 and rows 4*quad .. +3 of
        // the wave's 16; the score and dP products take turns, every row fragment serves both key halves
        auto score_tile = [&](const unsigned char* buffer, unsigned char* exchange) {
            const unsigned char* q_latent = buffer + L::Q_LATENT;
            const unsigned char* q_rope = buffer + L::Q_ROPE;
            const unsigned char* do_rows = buffer + L::DO_ROWS;
            const float* lse2 = reinterpret_cast<const float*>(buffer + L::STATS);
            const float* delta = lse2 + TILE;
            const int* token_of = reinterpret_cast<const int*>(delta + TILE);
            f32x4 s_acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            f32x4 dp_acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            bf16x8 ring[AHEAD];
            auto row_fragment = [&](auto tag) {
                constexpr int I = decltype(tag)::value;
                if constexpr (I >= 2 * O_STEPS) {
                    return quadrant_fragment<I - 2 * O_STEPS>(q_rope, narrow_quadrant);
                } else if constexpr (I % 2 == 0) {
                    return quadrant_fragment<I / 2>(q_latent, wide_quadrant);
                } else {
                    return quadrant_fragment<I / 2>(do_rows, wide_quadrant);
                }
            };
            fill_ring(ring, row_fragment);
            fragment_stream<Q_STEPS + O_STEPS>(ring, row_fragment, [&](auto tag, const bf16x8& fragment) {
                constexpr int I = decltype(tag)::value;
#pragma unroll
                for (int kh = 0; kh < 2; ++kh) {
                    if constexpr (I >= 2 * O_STEPS) {
                        s_acc[kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, kf[kh][I - O_STEPS], s_acc[kh], 0, 0, 0);
                    } else if constexpr (I % 2 == 0) {
                        s_acc[kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, kf[kh][I / 2], s_acc[kh], 0, 0, 0);
                    } else {
                        dp_acc[kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, kf[kh][I / 2], dp_acc[kh], 0, 0, 0);
                    }
                }
                if constexpr (I % 2 == 0) request(std::integral_constant<int, I / 2>{});
            });
            const int local = 16 * half + 4 * quad;
            const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse2 + local);
            const f32x4 delta4 = *reinterpret_cast<const f32x4*>(delta + local);
            const u32x4 token4 = *reinterpret_cast<const u32x4*>(token_of + local);
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                const int own_key = k0 + 16 * kh + l16;
                float p[4], ds[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[kh][i], c, -lse4[i]));
                    if (own_key > (int)token4[i]) probability = 0.f;
                    p[i] = probability;
                    ds[i] = probability * (dp_acc[kh][i] - delta4[i]) * scale;
                }
                exchange_store(exchange, 16 * kh + l16, local, p);     // [key][row]
                exchange_store(exchange + EXCHANGE_BYTES, 16 * kh + l16, local, ds);
            }
        };

        // One step of a gradient wave: the held fragments (tile t - 1) meet P and dS of that tile, and each gives way
        // to the same fragment of tile t in `buffer`.  Per 16-row step n: the query columns of the wave's eight
        // latent blocks (with dS), its rope block (with dS), the dO columns of the latent blocks (with P):
        // neighbouring products go to different accumulators.
        auto add_tile = [&](const unsigned char* buffer, const unsigned char* exchange, bool any) {
            const unsigned char* q_latent = buffer + L::Q_LATENT;
            const unsigned char* q_rope = buffer + L::Q_ROPE;
            const unsigned char* do_rows = buffer + L::DO_ROWS;
            bf16x8 pf[2], dsf[2];
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                pf[n] = dsf[n] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
                if (any) {
                    pf[n] = exchange_fragment(exchange, lq, g, n);
                    dsf[n] = exchange_fragment(exchange + EXCHANGE_BYTES, lq, g, n);
                }
            }
            static_for<0, 2 * PER_STEP>([&](auto tag) {
                constexpr int I = decltype(tag)::value;
                constexpr int N = I / PER_STEP;
                constexpr int F = I % PER_STEP;
                if constexpr (F < LATENT_BLOCKS) {
                    latent_acc[F] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[N], held[I], latent_acc[F], 0, 0, 0);
                    held[I] = transposed_fragment(q_latent, wide_columns.low[F % 4], wide_columns.high[F % 4],
                                                  N * 16 * Wide::ROW + 256 * (F / 4));
                } else if constexpr (F == LATENT_BLOCKS) {
                    rope_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[N], held[I], rope_acc, 0, 0, 0);
                    held[I] = transposed_fragment(q_rope, rope_columns_low, rope_columns_high, N * 16 * Narrow::ROW);
                } else {
                    constexpr int J = F - LATENT_BLOCKS - 1;
                    latent_acc[J] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[N], held[I], latent_acc[J], 0, 0, 0);
                    held[I] = transposed_fragment(do_rows, wide_columns.low[J % 4], wide_columns.high[J % 4],
                                                  N * 16 * Wide::ROW + 256 * (J / 4));
                }
                if constexpr (I % 2 == 0) request(std::integral_constant<int, I / 2>{});
                __builtin_amdgcn_sched_barrier(0);
            });
        };

        // Step t: tile t is in buffer t % 2 (scored there, and picked up by the gradient waves for step t + 1), tile
        // t + 1 arrives in the other buffer.  One more step after the last tile lets the gradient waves catch up.
        // Every step ends with a barrier behind all LDS reads, so the buffers are free when a segment begins.
        begin_requests(first_tile, 0);
        static_for<0, REQUESTS>(request);
        wait_vector_memory<0>();
        place_statistics(0);
        workgroup_barrier();

        for (int tile = first_tile; tile <= end_tile; ++tile) {
            const int parity = (tile - first_tile) & 1;
            const bool more = tile + 1 < end_tile;
            begin_requests(more ? tile + 1 : end_tile - 1, parity ^ 1);
            if constexpr (SCORES) {
                if (tile < end_tile) {
                    score_tile(lds + parity * L::BUFFER_BYTES, lds + L::EXCHANGE + parity * L::EXCHANGE_PAIR);
                }
            } else {
                add_tile(lds + parity * L::BUFFER_BYTES, lds + L::EXCHANGE + (parity ^ 1) * L::EXCHANGE_PAIR,
                         tile > first_tile);
            }
            wait_vector_memory<0>();
            place_statistics(parity ^ 1);
            workgroup_barrier();   // tile t has been read, P and dS of it and tile t + 1 are in place
        }

        // gradient waves: lane holds column (block, lq) and keys k0 + 8*(i/4) + 4*g + i%4
        if constexpr (!SCORES) {
            if (whole) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int k = k0 + 8 * (i / 4) + 4 * g + i % 4;
                    if (k < T) {
                        __bf16* latent_row = reinterpret_cast<__bf16*>(kv_latent_gradient) + ((size_t)batch * T + k) * RANK;
#pragma unroll
                        for (int j = 0; j < LATENT_BLOCKS; ++j) {
                            latent_row[32 * (LATENT_BLOCKS * half + j) + lq] = (__bf16)latent_acc[j][i];
                        }
                        __bf16* rope_row = reinterpret_cast<__bf16*>(key_rope_gradient) + ((size_t)batch * T + k) * ROPE;
                        rope_row[32 * half + lq] = (__bf16)rope_acc[i];
                    }
                }
            } else {
                const long long slot_number =
                    interval_length > 0 ? item : (long long)blockIdx.x + (long long)batch * visits.key_blocks + key_block;
                float* slot = partial_slots + slot_number * PARTIAL_FLOATS;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float* slot_row = slot + (8 * (i / 4) + 4 * g + i % 4) * WIDTH;
#pragma unroll
                    for (int j = 0; j < LATENT_BLOCKS; ++j) slot_row[32 * (LATENT_BLOCKS * half + j) + lq] = latent_acc[j][i];
                    slot_row[RANK + 32 * half + lq] = rope_acc[i];
                }
            }
        }
        position = batch * per_batch + segment_end;
    }
}

__global__ __launch_bounds__(THREADS) void mla_absorbed_key_gradient_kernel(
    bf16_t* __restrict__ kv_latent_gradient, bf16_t* __restrict__ key_rope_gradient, float* __restrict__ partial_slots,
    const float* __restrict__ delta_of_rows, const bf16_t* __restrict__ output_gradient,
    const float* __restrict__ logsumexp, const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int batch_size, int sequence_length,
    int heads, int ranges, int interval_length, float scale) {
    if (threadIdx.x < THREADS / 2) {
        key_gradient_walk<true>(kv_latent_gradient, key_rope_gradient, partial_slots, delta_of_rows, output_gradient,
                                logsumexp, query_latent, query_rope, kv_latent, key_rope, batch_size, sequence_length,
                                heads, ranges, interval_length, scale);
    } else {
        key_gradient_walk<false>(kv_latent_gradient, key_rope_gradient, partial_slots, delta_of_rows, output_gradient,
                                 logsumexp, query_latent, query_rope, kv_latent, key_rope, batch_size, sequence_length,
                                 heads, ranges, interval_length, scale);
    }
}

// ---- key gradients of inputs that outgrow the caches: 64 keys per workgroup ------
//
// There the kernel above is bound by what it moves: a row tile of 68 KB meets 32 keys.  This one has the same layout
// (score waves, gradient waves one tile behind that hold the tile's column fragments in registers, two 32-row
// buffers, one barrier a step) with 64 keys, so every row fetched does twice the work and a step carries twice the
// products for the same barrier, first reads and wait for the rows.  The gradient waves hold the latent sums of all
// 64 keys, 256 registers: all the accumulation registers a wave has (with more the compiler keeps sums in both
// register files and moves them inside the loop, waiting for every product it moves), besides 128 registers of held
// fragments.  The rope columns are therefore summed by the score waves.  Score wave w takes all 32 rows against keys
// 32w .. 32w + 31 (the keys as register operands, 144 registers; with the rows split instead each wave would hold all
// 64 keys, 288, and spill), so dS of its keys over the whole tile are its own: it reads them back from the exchange
// tile behind its own stores, which the LDS keeps in order, and multiplies them with the rope column blocks.
// Only the interval cut uses it: a workgroup walks one item.
struct KeyPairLayout {
    static constexpr int KEYS = 64;
    static constexpr int Q_LATENT = 0;                                   // [32 rows][512]
    static constexpr int DO_ROWS = Q_LATENT + Tile32<RANK>::BYTES;       // [32 rows][512]
    static constexpr int Q_ROPE = DO_ROWS + Tile32<RANK>::BYTES;         // [32 rows][64]
    static constexpr int STATS = Q_ROPE + Tile32<ROPE>::BYTES;
    static constexpr int BUFFER_BYTES = STATS + 3 * TILE * 4;
    static constexpr int EXCHANGE = 2 * BUFFER_BYTES;                    // the tile in use and the one arriving
    static constexpr int EXCHANGE_PART = (KEYS / TILE) * EXCHANGE_BYTES; // P (or dS) of a tile: [64 keys][32 rows]
    static constexpr int EXCHANGE_PAIR = 2 * EXCHANGE_PART;
    static constexpr int LDS_BYTES = EXCHANGE + 2 * EXCHANGE_PAIR;       // of the tile being scored and the one before
};
static_assert(KeyPairLayout::LDS_BYTES <= 160 * 1024, "LDS of a compute unit");

template <bool SCORES>
__device__ __forceinline__ void key_pair_walk(
    bf16_t* __restrict__ kv_latent_gradient, bf16_t* __restrict__ key_rope_gradient, float* __restrict__ partial_slots,
    const float* __restrict__ delta_of_rows, const bf16_t* __restrict__ output_gradient,
    const float* __restrict__ logsumexp, const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int sequence_length, int heads,
    int interval_length, float scale) {
    using L = KeyPairLayout;
    using Wide = Tile32<RANK>;
    using Narrow = Tile32<ROPE>;
    constexpr int Q_STEPS = WIDTH / 32;    // 18
    constexpr int O_STEPS = RANK / 32;     // 16
    constexpr int AHEAD = 6;
    constexpr int KEY_TILES = L::KEYS / TILE;
    constexpr int LATENT_BLOCKS = 8;       // per gradient wave
    constexpr int PER_STEP = 2 * LATENT_BLOCKS;   // column fragments per 16-row step of a gradient wave
    constexpr int ROWS_PER_WAVE = TILE / 4;
    constexpr int REQUESTS = 2 * ROWS_PER_WAVE + 1;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    __builtin_assume(tid >= 0 && tid < THREADS);
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int T = sequence_length;
    const long long rows = (long long)T * heads;
    const float c = scale * LOG2E;
    const int half = wave % 2;             // score waves: keys 32*half .. +31; gradient waves: column blocks 8*half .. +7
    const int l16 = lane % 16;
    const int quad = lane / 16;
    const QuadrantAt<RANK> wide_quadrant(lane, 0);
    const QuadrantAt<ROPE> narrow_quadrant(lane, 0);
    const TransposedAt<RANK> wide_columns(lane, 512 * half);
    const TransposedAt<ROPE> rope_columns(lane, 0);

    const unsigned lds_base = lds_offset_of(lds);
    unsigned wide_part[ROWS_PER_WAVE];
#pragma unroll
    for (int j = 0; j < ROWS_PER_WAVE; ++j) {
        wide_part[j] = 16u * (unsigned)(lane ^ index_math::tile_swizzle<Wide::ROW>(ROWS_PER_WAVE * wave + j));
    }
    const int narrow_row = ROWS_PER_WAVE * wave + lane / 8;
    const unsigned narrow_part = 16u * (unsigned)((lane % 8) ^ index_math::tile_swizzle<Narrow::ROW>(narrow_row));

    // the workgroup's item: the tiles of one key block inside one interval
    const index_math::KeyVisits visits = index_math::key_visits(T, heads, KEY_TILES);
    const index_math::KeyIntervals cut = index_math::key_intervals(T, heads, interval_length, KEY_TILES);
    const long long items = cut.items();
    const long long item = blockIdx.x;
    const int batch = (int)(item / items);
    int interval, key_block;
    cut.locate(item - batch * items, interval, key_block);
    const int first_tile = max(interval * interval_length, visits.first_tile(key_block));
    const int end_tile = cut.end_of(interval);
    const bool whole = first_tile == visits.first_tile(key_block) && end_tile == visits.row_tiles;

    const int k0 = key_block * L::KEYS;
    const long long batch_row0 = (long long)batch * rows;
    const bf16_t* ql = query_latent + batch_row0 * RANK;
    const bf16_t* qr = query_rope + batch_row0 * ROPE;
    const bf16_t* dout = output_gradient + batch_row0 * RANK;
    const bf16_t* latent = kv_latent + (size_t)batch * T * RANK;
    const bf16_t* rope = key_rope + (size_t)batch * T * ROPE;
    const float* lse_batch = logsumexp + (size_t)batch * heads * T;

    // score waves: the wave's 32 keys as B operands (column = key 32*half + 16*kh + l16), and their rope sums
    bf16x8 kf[2][Q_STEPS];
    f32x16 rope_acc[ROPE / 32];
    if constexpr (SCORES) {
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
            const int own_key = k0 + 32 * half + 16 * kh + l16;
            const size_t k = own_key < T ? own_key : 0;
            fetch_quadrant_operand(kf[kh], latent + k * RANK, rope + k * ROPE, own_key < T, quad);
        }
#pragma unroll
        for (int b = 0; b < ROPE / 32; ++b) clear(rope_acc[b]);
    }
    // gradient waves: latent column blocks 8*half + j of both key tiles, and the column fragments of the tile before
    // the one in LDS (zero before the first: its products add nothing)
    f32x16 latent_acc[KEY_TILES][LATENT_BLOCKS];
    bf16x8 held[2 * PER_STEP];
    if constexpr (!SCORES) {
#pragma unroll
        for (int kt = 0; kt < KEY_TILES; ++kt) {
#pragma unroll
            for (int j = 0; j < LATENT_BLOCKS; ++j) clear(latent_acc[kt][j]);
        }
#pragma unroll
        for (int f = 0; f < 2 * PER_STEP; ++f) held[f] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
    }

    struct {
        const bf16_t* latent;
        const bf16_t* gradient;
        const bf16_t* rope;
        int last_valid;
        unsigned buffer;
    } arriving;
    RowStatistics statistics = {0.f, 0.f, -1};
    auto begin_requests = [&](int tile, int parity) {
        const long long row0 = (long long)tile * TILE;
        arriving.latent = ql + row0 * RANK;
        arriving.gradient = dout + row0 * RANK;
        arriving.rope = qr + row0 * ROPE;
        arriving.last_valid = (int)min(rows - row0, (long long)TILE) - 1;
        arriving.buffer = lds_base + parity * L::BUFFER_BYTES;
        // the statistics of its rows: one lane per row, in a gradient wave (the score waves have more to do)
        if (tid >= 2 * 64 && tid < 2 * 64 + TILE) {
            const int r = tid - 2 * 64;
            statistics = {0.f, 0.f, -1};
            if (r <= arriving.last_valid) {
                int token, head;
                if (rows <= 0x7fffffffLL) {
                    const unsigned row = (unsigned)row0 + (unsigned)r;
                    token = (int)(row / (unsigned)heads);
                    head = (int)(row % (unsigned)heads);
                } else {
                    token = (int)((row0 + r) / heads);
                    head = (int)((row0 + r) % heads);
                }
                statistics.lse = lse_batch[(size_t)head * T + token];
                statistics.delta = delta_of_rows[(batch_row0 + row0 + r) * DELTA_STRIDE];
                statistics.token = token;
            }
        }
    };
    auto request = [&](auto tag) {
        constexpr int R = decltype(tag)::value;
        if constexpr (R < 2 * ROWS_PER_WAVE) {
            constexpr int J = R / 2;
            const int row = ROWS_PER_WAVE * wave + J;
            const unsigned source = wide_part[J] + (unsigned)(min(row, arriving.last_valid) * Wide::ROW);
            if constexpr (R % 2 == 0) {
                direct_load_16_offset(arriving.latent, source, arriving.buffer + L::Q_LATENT + row * Wide::ROW);
            } else {
                direct_load_16_offset(arriving.gradient, source, arriving.buffer + L::DO_ROWS + row * Wide::ROW);
            }
        } else if constexpr (R == 2 * ROWS_PER_WAVE) {
            direct_load_16_offset(arriving.rope, narrow_part + (unsigned)(min(narrow_row, arriving.last_valid) * Narrow::ROW),
                                  arriving.buffer + L::Q_ROPE + ROWS_PER_WAVE * wave * Narrow::ROW);
        }
    };
    auto place_statistics = [&](int parity) {
        if (tid >= 2 * 64 && tid < 2 * 64 + TILE) {
            const int r = tid - 2 * 64;
            float* lse2 = reinterpret_cast<float*>(lds + parity * L::BUFFER_BYTES + L::STATS);
            lse2[r] = statistics.lse * LOG2E;
            lse2[TILE + r] = statistics.delta;
            reinterpret_cast<int*>(lse2)[2 * TILE + r] = statistics.token;
        }
    };

    // scores of one tile: (rows x keys) blocks of 16 x 16, lane holds key 32*half + 16*kh + l16 and rows 16*r + 4*quad .. +3;
    // the two halves of the rows one after the other, every row fragment serves both key blocks
    auto score_tile = [&](const unsigned char* buffer, unsigned char* exchange) {
        const unsigned char* q_latent = buffer + L::Q_LATENT;
        const unsigned char* q_rope = buffer + L::Q_ROPE;
        const unsigned char* do_rows = buffer + L::DO_ROWS;
        const float* lse2 = reinterpret_cast<const float*>(buffer + L::STATS);
        const float* delta = lse2 + TILE;
        const int* token_of = reinterpret_cast<const int*>(delta + TILE);
        f32x4 s_acc[2][2], dp_acc[2][2];   // [half of the rows][key block]
#pragma unroll
        for (int r = 0; r < 2; ++r) {
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) s_acc[r][kh] = dp_acc[r][kh] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        constexpr int PER_HALF = Q_STEPS + O_STEPS;
        bf16x8 ring[AHEAD];
        auto row_fragment = [&](auto tag) {
            constexpr int R = decltype(tag)::value / PER_HALF;
            constexpr int I = decltype(tag)::value % PER_HALF;
            if constexpr (I >= 2 * O_STEPS) {
                return quadrant_fragment<I - 2 * O_STEPS>(q_rope + R * 16 * Narrow::ROW, narrow_quadrant);
            } else if constexpr (I % 2 == 0) {
                return quadrant_fragment<I / 2>(q_latent + R * 16 * Wide::ROW, wide_quadrant);
            } else {
                return quadrant_fragment<I / 2>(do_rows + R * 16 * Wide::ROW, wide_quadrant);
            }
        };
        fill_ring(ring, row_fragment);
        fragment_stream<2 * PER_HALF>(ring, row_fragment, [&](auto tag, const bf16x8& fragment) {
            constexpr int R = decltype(tag)::value / PER_HALF;
            constexpr int I = decltype(tag)::value % PER_HALF;
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                if constexpr (I >= 2 * O_STEPS) {
                    s_acc[R][kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, kf[kh][I - O_STEPS], s_acc[R][kh], 0, 0, 0);
                } else if constexpr (I % 2 == 0) {
                    s_acc[R][kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, kf[kh][I / 2], s_acc[R][kh], 0, 0, 0);
                } else {
                    dp_acc[R][kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fragment, kf[kh][I / 2], dp_acc[R][kh], 0, 0, 0);
                }
            }
            if constexpr (decltype(tag)::value % 4 == 0) request(std::integral_constant<int, decltype(tag)::value / 4>{});
        });
        // the rope columns of the tile's rows, for the rope products below
        bf16x8 rope_columns_of_rows[2][ROPE / 32];
#pragma unroll
        for (int n = 0; n < 2; ++n) {
#pragma unroll
            for (int b = 0; b < ROPE / 32; ++b) {
                rope_columns_of_rows[n][b] = transposed_fragment(q_rope, rope_columns.low[b], rope_columns.high[b], n * 16 * Narrow::ROW);
            }
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int local = 16 * r + 4 * quad;
            const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse2 + local);
            const f32x4 delta4 = *reinterpret_cast<const f32x4*>(delta + local);
            const u32x4 token4 = *reinterpret_cast<const u32x4*>(token_of + local);
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                const int own_key = k0 + 32 * half + 16 * kh + l16;
                float p[4], ds[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[r][kh][i], c, -lse4[i]));
                    if (own_key > (int)token4[i]) probability = 0.f;
                    p[i] = probability;
                    ds[i] = probability * (dp_acc[r][kh][i] - delta4[i]) * scale;
                }
                // [key][row], the wave's 32 keys are one part of EXCHANGE_BYTES
                exchange_store(exchange + half * EXCHANGE_BYTES, 16 * kh + l16, local, p);
                exchange_store(exchange + L::EXCHANGE_PART + half * EXCHANGE_BYTES, 16 * kh + l16, local, ds);
            }
        }
        // dK_rope += dS^T Q_rope for the wave's keys: their dS of all 32 rows were written by this wave
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const bf16x8 gradient = exchange_fragment(exchange + L::EXCHANGE_PART + half * EXCHANGE_BYTES, lq, g, n);
#pragma unroll
            for (int b = 0; b < ROPE / 32; ++b) {
                rope_acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gradient, rope_columns_of_rows[n][b], rope_acc[b], 0, 0, 0);
            }
        }
    };

    // One step of a gradient wave: the held fragments (tile t - 1) meet P and dS of that tile, both key tiles one after
    // the other, and each gives way to the same fragment of tile t in `buffer`.  Per 16-row step n: the query columns
    // of the wave's eight latent blocks (with dS), then the dO columns of the same blocks (with P).
    auto add_tile = [&](const unsigned char* buffer, const unsigned char* exchange, bool any) {
        const unsigned char* q_latent = buffer + L::Q_LATENT;
        const unsigned char* do_rows = buffer + L::DO_ROWS;
        bf16x8 pf[KEY_TILES][2], dsf[KEY_TILES][2];
#pragma unroll
        for (int kt = 0; kt < KEY_TILES; ++kt) {
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                pf[kt][n] = dsf[kt][n] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
                if (any) {
                    pf[kt][n] = exchange_fragment(exchange + kt * EXCHANGE_BYTES, lq, g, n);
                    dsf[kt][n] = exchange_fragment(exchange + L::EXCHANGE_PART + kt * EXCHANGE_BYTES, lq, g, n);
                }
            }
        }
        static_for<0, 2 * PER_STEP>([&](auto tag) {
            constexpr int I = decltype(tag)::value;
            constexpr int N = I / PER_STEP;
            constexpr int F = I % PER_STEP;
            if constexpr (F < LATENT_BLOCKS) {
#pragma unroll
                for (int kt = 0; kt < KEY_TILES; ++kt) {
                    latent_acc[kt][F] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[kt][N], held[I], latent_acc[kt][F], 0, 0, 0);
                }
                held[I] = transposed_fragment(q_latent, wide_columns.low[F % 4], wide_columns.high[F % 4],
                                              N * 16 * Wide::ROW + 256 * (F / 4));
            } else {
                constexpr int J = F - LATENT_BLOCKS;
#pragma unroll
                for (int kt = 0; kt < KEY_TILES; ++kt) {
                    latent_acc[kt][J] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[kt][N], held[I], latent_acc[kt][J], 0, 0, 0);
                }
                held[I] = transposed_fragment(do_rows, wide_columns.low[J % 4], wide_columns.high[J % 4],
                                              N * 16 * Wide::ROW + 256 * (J / 4));
            }
            if constexpr (I % 2 == 0) request(std::integral_constant<int, I / 2>{});
            if constexpr (I + 1 == 2 * PER_STEP) request(std::integral_constant<int, PER_STEP>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // Step t: tile t is in buffer t % 2 (scored there, and picked up by the gradient waves for step t + 1), tile
    // t + 1 arrives in the other buffer.  One more step after the last tile lets the gradient waves catch up.
    begin_requests(first_tile, 0);
    static_for<0, REQUESTS>(request);
    wait_vector_memory<0>();
    place_statistics(0);
    workgroup_barrier();

    for (int tile = first_tile; tile <= end_tile; ++tile) {
        const int parity = (tile - first_tile) & 1;
        const bool more = tile + 1 < end_tile;
        begin_requests(more ? tile + 1 : end_tile - 1, parity ^ 1);
        if constexpr (SCORES) {
            if (tile < end_tile) {
                score_tile(lds + parity * L::BUFFER_BYTES, lds + L::EXCHANGE + parity * L::EXCHANGE_PAIR);
            }
        } else {
            add_tile(lds + parity * L::BUFFER_BYTES, lds + L::EXCHANGE + (parity ^ 1) * L::EXCHANGE_PAIR, tile > first_tile);
        }
        wait_vector_memory<0>();
        place_statistics(parity ^ 1);
        workgroup_barrier();   // tile t has been read, P and dS of it and tile t + 1 are in place
    }

    // lane holds column (block, lq) and keys (first of the 32) + 8*(i/4) + 4*g + i%4: score wave w of keys 32w .. +31 and
    // the two rope blocks, the gradient waves of both key tiles and their eight latent blocks
    float* slot = partial_slots + item * (KEY_TILES * PARTIAL_FLOATS);   // [64 keys][576]
    if constexpr (SCORES) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int key = TILE * half + 8 * (i / 4) + 4 * g + i % 4;
            if (whole) {
                if (k0 + key < T) {
                    __bf16* rope_row = reinterpret_cast<__bf16*>(key_rope_gradient) + ((size_t)batch * T + k0 + key) * ROPE;
#pragma unroll
                    for (int b = 0; b < ROPE / 32; ++b) rope_row[32 * b + lq] = (__bf16)rope_acc[b][i];
                }
            } else {
#pragma unroll
                for (int b = 0; b < ROPE / 32; ++b) slot[key * WIDTH + RANK + 32 * b + lq] = rope_acc[b][i];
            }
        }
    } else {
#pragma unroll
        for (int kt = 0; kt < KEY_TILES; ++kt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = TILE * kt + 8 * (i / 4) + 4 * g + i % 4;
                if (whole) {
                    if (k0 + key < T) {
                        __bf16* latent_row = reinterpret_cast<__bf16*>(kv_latent_gradient) + ((size_t)batch * T + k0 + key) * RANK;
#pragma unroll
                        for (int j = 0; j < LATENT_BLOCKS; ++j) {
                            latent_row[32 * (LATENT_BLOCKS * half + j) + lq] = (__bf16)latent_acc[kt][j][i];
                        }
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < LATENT_BLOCKS; ++j) {
                        slot[key * WIDTH + 32 * (LATENT_BLOCKS * half + j) + lq] = latent_acc[kt][j][i];
                    }
                }
            }
        }
    }
}

__global__ __launch_bounds__(THREADS) void mla_absorbed_key_pair_gradient_kernel(
    bf16_t* __restrict__ kv_latent_gradient, bf16_t* __restrict__ key_rope_gradient, float* __restrict__ partial_slots,
    const float* __restrict__ delta_of_rows, const bf16_t* __restrict__ output_gradient,
    const float* __restrict__ logsumexp, const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int sequence_length, int heads,
    int interval_length, float scale) {
    if (threadIdx.x < THREADS / 2) {
        key_pair_walk<true>(kv_latent_gradient, key_rope_gradient, partial_slots, delta_of_rows, output_gradient, logsumexp,
                                 query_latent, query_rope, kv_latent, key_rope, sequence_length, heads, interval_length, scale);
    } else {
        key_pair_walk<false>(kv_latent_gradient, key_rope_gradient, partial_slots, delta_of_rows, output_gradient, logsumexp,
                                  query_latent, query_rope, kv_latent, key_rope, sequence_length, heads, interval_length, scale);
    }
}

// Sums the partial key gradients of every key block whose visits were cut, in range (or interval) order.  Workgroup (x, y)
// takes the y-th 1/REDUCTION_PARTS of key block x (numbered through the batch elements), a thread four
// neighbouring columns of one key; a block that one range held whole wrote its gradients itself.
constexpr int REDUCTION_PARTS = PARTIAL_FLOATS / 4 / THREADS;   // 18
static_assert(REDUCTION_PARTS * THREADS * 4 == PARTIAL_FLOATS, "slot size");

__global__ __launch_bounds__(THREADS) void mla_absorbed_key_reduction_kernel(
    bf16_t* __restrict__ kv_latent_gradient, bf16_t* __restrict__ key_rope_gradient,
    const float* __restrict__ partial_slots, int sequence_length, int heads, int batch_size, int ranges,
    int interval_length, int key_tiles) {
    // key blocks and slots of 32 * key_tiles keys, blockIdx.y up to REDUCTION_PARTS * key_tiles
    const index_math::KeyVisits visits = index_math::key_visits(sequence_length, heads, key_tiles);
    const long long slot_floats = (long long)key_tiles * PARTIAL_FLOATS;
    const int batch = blockIdx.x / visits.key_blocks;
    const int key_block = blockIdx.x % visits.key_blocks;
    const int index = blockIdx.y * THREADS + threadIdx.x;   // which four floats of the slot
    f32x4 sum;
    if (interval_length > 0) {
        // the block's items: one per interval from the one its first tile lies in, slot = item number
        const index_math::KeyIntervals cut = index_math::key_intervals(sequence_length, heads, interval_length, key_tiles);
        const int first = cut.first_interval(key_block);
        if (first == cut.intervals - 1) return;
        long long slot = batch * cut.items() + cut.items_before(first) + key_block;
        sum = *reinterpret_cast<const f32x4*>(partial_slots + slot * slot_floats + 4 * index);
        // eight parts per round trip, added in the order of the intervals (one at a time, a block with 64 parts
        // waited for 64 round trips in a row)
        constexpr int TOGETHER = 8;
        for (int interval = first + 1; interval < cut.intervals; interval += TOGETHER) {
            f32x4 value[TOGETHER];
#pragma unroll
            for (int j = 0; j < TOGETHER; ++j) {
                value[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (interval + j < cut.intervals) {
                    slot += cut.blocks_in(interval + j - 1);
                    value[j] = *reinterpret_cast<const f32x4*>(partial_slots + slot * slot_floats + 4 * index);
                }
            }
#pragma unroll
            for (int j = 0; j < TOGETHER; ++j) {
#pragma unroll
                for (int e = 0; e < 4; ++e) sum[e] += value[j][e];
            }
        }
    } else {
        const long long per_batch = visits.per_batch();
        const long long total = per_batch * batch_size;
        const long long begin = batch * per_batch + visits.before(key_block);
        const long long end = batch * per_batch + visits.before(key_block + 1);
        const long long first_range = index_math::wide_range_of(total, ranges, begin);
        const long long last_range = index_math::wide_range_of(total, ranges, end - 1);
        if (first_range == last_range) return;
        const float* first_slot = partial_slots + (first_range + blockIdx.x) * slot_floats + 4 * index;
        const int parts = (int)(last_range - first_range) + 1;
        sum = *reinterpret_cast<const f32x4*>(first_slot);
        constexpr int TOGETHER = 8;
        for (int part = 1; part < parts; part += TOGETHER) {
            f32x4 value[TOGETHER];
#pragma unroll
            for (int j = 0; j < TOGETHER; ++j) {
                value[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (part + j < parts) {
                    value[j] = *reinterpret_cast<const f32x4*>(first_slot + (long long)(part + j) * slot_floats);
                }
            }
#pragma unroll
            for (int j = 0; j < TOGETHER; ++j) {
#pragma unroll
                for (int e = 0; e < 4; ++e) sum[e] += value[j][e];
            }
        }
    }
    const int key = key_block * TILE * key_tiles + (4 * index) / WIDTH;
    const int column = (4 * index) % WIDTH;
    if (key < sequence_length) {
        u32x2 packed;
        packed.x = pack_bf16(sum[0], sum[1]);
        packed.y = pack_bf16(sum[2], sum[3]);
        bf16_t* destination = column < RANK
            ? kv_latent_gradient + ((size_t)batch * sequence_length + key) * RANK + column
            : key_rope_gradient + ((size_t)batch * sequence_length + key) * ROPE + (column - RANK);
        *reinterpret_cast<u32x2*>(destination) = packed;
    }
}

template <typename Kernel>
void raise_lds_limit(Kernel kernel, int bytes) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  bytes));
}

constexpr long long LARGE_INPUT_BYTES = 64LL << 20;   // per batch element, against 32 MB of L2 and 256 MB behind it

// mla_absorbed_backward_set_key_interval_tiles (> 0) forces the interval cut with that many row tiles per interval at
// any size the slots allow; 0 gives the choice back to the dispatch below.
std::atomic<int> forced_key_interval_tiles{0};

int forced_interval_tiles() {
    return forced_key_interval_tiles.load(std::memory_order_relaxed);
}

int device_compute_units() {
    return hip_common::compute_units_of_current_device();
}

}  // namespace

void mla_absorbed_backward_set_key_interval_tiles(int tiles) {
    forced_key_interval_tiles.store(tiles > 0 && tiles < (1 << 24) ? tiles : 0, std::memory_order_relaxed);
}

void mla_absorbed_backward_dispatch(bf16_t* query_latent_gradient, bf16_t* query_rope_gradient,
                                    bf16_t* kv_latent_gradient, bf16_t* key_rope_gradient,
                                    const bf16_t* output_gradient, const bf16_t* output, const float* logsumexp,
                                    const bf16_t* query_latent, const bf16_t* query_rope, const bf16_t* kv_latent,
                                    const bf16_t* key_rope, int batch_size, int sequence_length, int heads, float scale,
                                    hipStream_t stream) {
    const long long rows = (long long)sequence_length * heads;
    const long long row_blocks = (rows + TILE - 1) / TILE;
    if (row_blocks * batch_size > 0x7fffffffLL) {
        throw std::invalid_argument("MLA backward: batch*tokens*heads exceeds the grid limit");
    }
    if (reinterpret_cast<uintptr_t>(query_latent_gradient) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(query_rope_gradient) % 16 != 0) {
        throw std::invalid_argument("MLA backward: the query gradients must be aligned to 16 bytes");
    }
    static hip_common::OncePerDevice prepared;
    prepared.run([] {
        raise_lds_limit(mla_absorbed_query_gradient_kernel, QueryGradLayout::LDS_BYTES);
        raise_lds_limit(mla_absorbed_key_gradient_kernel, KeyGradLayout::LDS_BYTES);
        raise_lds_limit(mla_absorbed_key_pair_gradient_kernel, KeyPairLayout::LDS_BYTES);
    });
    // scratch memory until the last launch: delta in the rope query gradients, partial key gradients in the latent ones
    float* delta = reinterpret_cast<float*>(query_rope_gradient);
    float* partial_slots = reinterpret_cast<float*>(query_latent_gradient);
    const index_math::KeyVisits visits = index_math::key_visits(sequence_length, heads);
    long long blocks = (long long)visits.key_blocks * batch_size;
    const long long total = visits.per_batch() * batch_size;
    const long long scratch_bytes = rows * batch_size * RANK * 2;
    // Rows that outgrow the caches (query and dO rows of a batch element, 2176 bytes per row): the interval cut
    // with key blocks of 64 keys (mla_absorbed_key_pair_gradient_kernel)
    constexpr int PAIR = KeyPairLayout::KEYS / TILE;
    int interval_length = 0;
    int key_tiles = 1;
    long long grid = 0;
    const int forced = forced_interval_tiles();
    if (forced > 0 || rows * (2 * RANK + ROPE) * 2 > LARGE_INPUT_BYTES) {
        const long long slots = scratch_bytes / (PAIR * index_math::KEY_PARTIAL_BYTES);
        // (the choice walks the intervals of several lengths: remembered for the shape a thread asked about last)
        struct Choice {
            int sequence_length = -1, heads = -1, batch_size = -1, units = -1, forced = -1, tiles = 0;
            long long items = 0;
            int key_blocks = 0;
        };
        static thread_local Choice last;
        const int units = device_compute_units();
        if (last.sequence_length != sequence_length || last.heads != heads || last.batch_size != batch_size ||
            last.units != units || last.forced != forced) {
            last = Choice{sequence_length, heads, batch_size, units, forced, 0, 0, 0};
            last.tiles = forced > 0 ? forced
                                    : index_math::key_interval_choice(sequence_length, heads, batch_size, slots, units, PAIR);
            if (last.tiles > 0) {
                const index_math::KeyIntervals chosen = index_math::key_intervals(sequence_length, heads, last.tiles, PAIR);
                last.items = chosen.items() * batch_size;
                last.key_blocks = chosen.key_blocks;
            }
        }
        const int tiles = last.tiles;
        const long long items = last.items;
        // a slot for each item
        if (tiles > 0 && items <= slots && items <= 0x7fffffffLL) {
            interval_length = tiles;
            key_tiles = PAIR;
            grid = items;
            blocks = (long long)last.key_blocks * batch_size;
        }
    }
    long long ranges = 0;
    if (interval_length == 0) {
        ranges = index_math::key_gradient_ranges(total, blocks, visits.row_tiles, scratch_bytes, device_compute_units());
        grid = ranges > 0 ? ranges : blocks;
    }

    hipLaunchKernelGGL(mla_absorbed_row_statistics_kernel, dim3((unsigned)(row_blocks * batch_size)), dim3(THREADS), 0,
                       stream, delta, output_gradient, output, rows * batch_size);
    HIP_CHECK(hipGetLastError());
    if (interval_length > 0) {
        hipLaunchKernelGGL(mla_absorbed_key_pair_gradient_kernel, dim3((unsigned)grid), dim3(THREADS),
                           KeyPairLayout::LDS_BYTES, stream, kv_latent_gradient, key_rope_gradient, partial_slots, delta,
                           output_gradient, logsumexp, query_latent, query_rope, kv_latent, key_rope, sequence_length,
                           heads, interval_length, scale);
    } else {
        hipLaunchKernelGGL(mla_absorbed_key_gradient_kernel, dim3((unsigned)grid), dim3(THREADS), KeyGradLayout::LDS_BYTES,
                           stream, kv_latent_gradient, key_rope_gradient, partial_slots, delta, output_gradient, logsumexp,
                           query_latent, query_rope, kv_latent, key_rope, batch_size, sequence_length, heads, (int)ranges,
                           0, scale);
    }
    HIP_CHECK(hipGetLastError());
    if (ranges > 0 || interval_length > 0) {
        hipLaunchKernelGGL(mla_absorbed_key_reduction_kernel, dim3((unsigned)blocks, REDUCTION_PARTS * key_tiles),
                           dim3(THREADS), 0, stream, kv_latent_gradient, key_rope_gradient, partial_slots, sequence_length,
                           heads, batch_size, (int)ranges, interval_length, key_tiles);
        HIP_CHECK(hipGetLastError());
    }
    const long long query_blocks = (rows + QUERY_ROWS - 1) / QUERY_ROWS;
    hipLaunchKernelGGL(mla_absorbed_query_gradient_kernel, dim3((unsigned)(query_blocks * batch_size)), dim3(QUERY_THREADS),
                       QueryGradLayout::LDS_BYTES, stream, query_latent_gradient, query_rope_gradient, delta,
                       output_gradient, logsumexp, query_latent, query_rope, kv_latent, key_rope, sequence_length, heads,
                       (int)query_blocks, scale);
    HIP_CHECK(hipGetLastError());
}

}  // namespace dscuda
