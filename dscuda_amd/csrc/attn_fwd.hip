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
// Tiles: global -> LDS without registers
//   K and V tiles arrive by global_load_lds (16 bytes per lane, 1 KB of
//   consecutive LDS per wave instruction), both row-major, two stages.  No
//   thread holds tile data in registers and nothing is written to LDS with
//   store instructions.  With no padding possible inside the 1 KB a wave
//   instruction fills, bank spread comes from a swizzle applied on the global
//   side (which 16-byte chunk a lane fetches):
//     K  : chunk c of row r sits at position c ^ fK(r).  A fragment read is 16
//          lanes x 16 B down a column of rows; fK(r) = (r>>1)&7 for rows that
//          are 128 (mod 256) bytes long, r&15 for rows that are 0 (mod 256).
//     V  : MFMA wants the contraction index (key) contiguous per lane, V has
//          d_v contiguous.  ds_read_b64_tr_b16 transposes a 4 keys x 16 columns
//          block across 16 lanes while reading, so the row-major tile is used
//          as it is.  Such a read touches 4 rows x 64 bytes; rows are 64*NG
//          bytes long (NG = d_v/32 column groups), so the 64-byte group index
//          of row r is XORed with r&3 (NG = 4) or (r>>1)&1 (NG = 2), and the
//          lane that addresses row r undoes it in its own address.
//   A tile is requested while the previous one is consumed; arrival is ordered
//   by s_waitcnt vmcnt + one workgroup barrier per tile.
#include "attn_kernels.h"
#include "hip_common.h"
#include "index_math.h"

#include <cmath>
#include <stdexcept>
#include <string>
#include <type_traits>

namespace dscuda {
namespace {

template <int DQK, int DV, int NWAVES>
struct FwdConfig {
    static constexpr int BN = 64;
    static constexpr int BM = 32 * NWAVES;
    static constexpr int THREADS = 64 * NWAVES;
    static constexpr int K_ROW = DQK * 2;                  // bytes
    static constexpr int K_CHUNKS = DQK / 8;               // 16-byte chunks per row
    static constexpr int K_BYTES = BN * K_ROW;
    static constexpr int V_ROW = DV * 2;
    static constexpr int V_CHUNKS = DV / 8;
    static constexpr int V_GROUPS = DV / 32;               // 64-byte column groups per row
    static constexpr int V_BYTES = BN * V_ROW;
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
    static constexpr int K_LOADS_PER_WAVE = K_BYTES / 1024 / NWAVES;   // wave instructions
    static constexpr int V_LOADS_PER_WAVE = V_BYTES / 1024 / NWAVES;
    static constexpr int O_PITCH = DV * 2 + 16;            // epilogue staging, bytes
    static constexpr int O_BYTES = BM * O_PITCH;
    static constexpr int LDS_BYTES = (2 * STAGE_BYTES > O_BYTES) ? 2 * STAGE_BYTES : O_BYTES;
    static_assert(K_BYTES % (1024 * NWAVES) == 0 && V_BYTES % (1024 * NWAVES) == 0,
                  "tile loads must divide evenly over the waves");
    static_assert(K_ROW % 128 == 0, "K rows must be a multiple of 128 bytes");
    static_assert(V_GROUPS == 2 || V_GROUPS == 4, "d_v must be 64 or 128");

    __device__ static constexpr int k_swizzle(int row) {
        return (K_ROW % 256 == 0) ? (row & 15) : ((row >> 1) & 7);
    }
    __device__ static constexpr int v_flip(int row) {
        return V_GROUPS == 4 ? (row & 3) : ((row >> 1) & 1);
    }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4* transposing_read_pointer;

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
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
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
    const unsigned k_stride_bytes = (unsigned)key_value_heads * DQK * 2;
    const unsigned v_stride_bytes = (unsigned)key_value_heads * DV * 2;
    const bf16_t* q_base = query + ((size_t)b * S * query_heads + h) * DQK;
    const unsigned char* k_base =
        reinterpret_cast<const unsigned char*>(key + ((size_t)b * S * key_value_heads + hk) * DQK);
    const unsigned char* v_base =
        reinterpret_cast<const unsigned char*>(value + ((size_t)b * S * key_value_heads + hk) * DV);

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
    const unsigned lds_base = lds_offset_of(lds);

    // Requests this wave's share of tile `tile` into `stage`.  Rows past the end
    // of the sequence are clamped to the last one: such keys are invisible to
    // every stored query, the data only has to be finite.
    auto request_tile = [&](int tile, int stage) {
        const int key0 = tile * BN;
        const int row_limit = S - 1 - key0;
        const unsigned char* k_tile = k_base + (size_t)key0 * k_stride_bytes;
        const unsigned char* v_tile = v_base + (size_t)key0 * v_stride_bytes;
        const unsigned stage_base = lds_base + stage * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::K_LOADS_PER_WAVE; ++i) {
            const int load = wave * C::K_LOADS_PER_WAVE + i;
            const int slot = 64 * load + lane;
            const int row = slot / C::K_CHUNKS;
            const int chunk = (slot % C::K_CHUNKS) ^ C::k_swizzle(row);
            const unsigned offset = (unsigned)min(row, row_limit) * k_stride_bytes + 16u * chunk;
            direct_load_16_offset(k_tile, offset, stage_base + load * 1024);
        }
#pragma unroll
        for (int i = 0; i < C::V_LOADS_PER_WAVE; ++i) {
            const int load = wave * C::V_LOADS_PER_WAVE + i;
            const int slot = 64 * load + lane;
            const int row = slot / C::V_CHUNKS;
            const int chunk = (slot % C::V_CHUNKS) ^ (C::v_flip(row) << 2);
            const unsigned offset = (unsigned)min(row, row_limit) * v_stride_bytes + 16u * chunk;
            direct_load_16_offset(v_tile, offset, stage_base + C::K_BYTES + load * 1024);
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

    // Per-lane pieces of the LDS read addresses.
    const int k_swz = C::k_swizzle(lq);                        // rows lq and lq+32 share it
    const int s16 = lane % 16;
    const int v_row = 4 * g + s16 / 4;                          // + 16*n, + 8 for the second read
    const int v_in_group = 32 * ((lane / 16) % 2) + 8 * (s16 % 4);
    const int v_flip = C::v_flip(v_row);                        // rows v_row + 8*m share it

    wait_vector_memory<0>();   // the query loads: no wait for them may remain inside the loop
    request_tile(0, 0);

    for (int tile = 0; tile < tiles; ++tile) {
        const int stage = tile & 1;
        wait_vector_memory<0>();   // this wave's share of the tile has landed
        workgroup_barrier();       // ... and everybody's; every wave has left the previous tile
        if (tile + 1 < tiles) {
            request_tile(tile + 1, stage ^ 1);
        }
        const int key0 = tile * BN;
        if (key0 <= wave_q0 + 31) {  // otherwise every key of the tile is in this wave's future
            const unsigned char* k_lds = lds + stage * C::STAGE_BYTES;
            const unsigned char* v_lds = k_lds + C::K_BYTES;

            f32x16 s_acc[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s_acc[mb][i] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const int position = (2 * ks + g) ^ k_swz;
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    const bf16x8 a =
                        *reinterpret_cast<const bf16x8*>(k_lds + (32 * mb + lq) * C::K_ROW + 16 * position);
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

            // V^T operand through transposing reads.  In a block of 16 lanes, lane s
            // points at key row 16n + 4g + s/4 (+8 for the second read) and columns
            // 4*(s%4)..+3 of the 16-column half (block%2) of column group d; the
            // instruction hands lane i column i of the four rows.  Together: MFMA row
            // lane%32, keys {4g..4g+3, 8+4g..8+4g+3} of the 16-key step, the k-order
            // P^T carries from the C layout.
#pragma unroll
            for (int n = 0; n < 4; ++n) {
#pragma unroll
                for (int d = 0; d < DBLOCKS; ++d) {
                    const unsigned char* first =
                        v_lds + (16 * n + v_row) * C::V_ROW + 64 * (d ^ v_flip) + v_in_group;
                    const s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)first);
                    const s16x4 high =
                        __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(first + 8 * C::V_ROW));
                    const s16x8 both = __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7);
                    o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf[n],
                                                                       o_acc[d], 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue: normalise, stage O through LDS for 16-byte row stores
    workgroup_barrier();   // every wave is done reading the tile stages
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

// ---------------------------------------------------------------------------
// Persistent two-phase ("ping-pong") variant for long sequences.
//
// One workgroup of 8 waves (2 per SIMD) per compute unit walks a list of work
// items, an item being one block of 256 queries of one (batch, head).
//
// Phases.  A SIMD's matrix pipeline idles while its waves run the softmax, and
// with one barrier per tile both waves of a SIMD run it at the same time.  Here
// every wave alternates between two phases that end in a workgroup barrier:
//     X(j): request later tiles, softmax of S(j) -> P(j)          (VALU, exp)
//     Y(j): O += V(j)^T P(j), then S(j+1) = K(j+1) Q^T            (MFMA, LDS reads)
// Waves 4..7 run one extra barrier before their first phase, so they are in X
// while waves 0..3 (the other wave of each SIMD) are in Y and the reverse: the
// matrix pipeline always has a wave feeding it.  Y raises its wave priority.
//
// Y is one stream of MFMAs (PV then QK), each with one A fragment from LDS.
// Fragments go through a ring of RING register sets that runs RING MFMAs ahead
// of their use; the first RING fragments (of V(j)) are read at the end of X(j),
// before the barrier, so that Y starts with its operands in registers.
//
// Tiles.  K tiles sit in a ring of three slots, V tiles in a ring of four, and
// the tiles of all items of a workgroup form one stream: a wave requests stream
// tile t+2 during X of stream tile t, whether it belongs to this item or to the
// next one, and waits for its own requests at the end of that tile's Y; the
// barrier that ends Y of the later group publishes them.  K(t+2) is first read
// in Y(t+1), V(t+2) at the end of X(t+2); the slots they overwrite (K(t-1),
// V(t-2)) were last read in Y(t-2).  So a new item finds its first two tiles in
// LDS; what stays exposed at an item switch is the load of the new queries.
//
// Work order.  Workgroup w belongs to cluster w % 8 (workgroups are dealt
// round-robin to the 8 XCDs, each with its own L2) and the (batch, head) pairs
// are dealt to the clusters the same way.  Inside a cluster the items are laid
// out two heads at a time, blocks from the heaviest (last) to the lightest, and
// cut into rounds of one item per workgroup; odd rounds are handed out in
// reverse, so a workgroup's heavy and light blocks add up to the same total
// while the cluster works on two heads at any time.
struct PingPong {
    static constexpr int K_SLOTS = 3;
    static constexpr int V_SLOTS = 4;
    static constexpr int RING = 8;
    static constexpr int CLUSTERS = 8;
    // Output rows leave through LDS, half a row (64 columns, one 128-byte line) at a time: 32 rows of
    // 128 + 16 bytes per wave, for the four waves of one group (the two groups store in different phases).
    static constexpr int O_HALF_COLUMNS = 64;
    static constexpr int O_PITCH = O_HALF_COLUMNS * 2 + 16;
    static constexpr int O_WAVE_BYTES = 32 * O_PITCH;
    static constexpr int O_BYTES = 4 * O_WAVE_BYTES;
};

using index_math::forward_item;
using index_math::ForwardItem;

template <int DQK, int DV>
__global__ __launch_bounds__(512) void attention_forward_pingpong_kernel(
    bf16_t* __restrict__ output, float* __restrict__ logsumexp,
    const bf16_t* __restrict__ query, const bf16_t* __restrict__ key, const bf16_t* __restrict__ value,
    int sequence_length, int query_heads, int key_value_heads, int query_blocks, int batch_heads, int clusters,
    float scale) {
    using C = FwdConfig<DQK, DV, 8>;
    constexpr int BN = C::BN;
    constexpr int KSTEPS = DQK / 16;
    constexpr int DBLOCKS = DV / 32;
    constexpr int SPAN = (C::K_ROW % 256 == 0) ? 16 : 8;   // chunk positions the K swizzle permutes
    constexpr int KLOW = SPAN / 2;                          // k-steps with distinct swizzled addresses
    constexpr int V_RING = PingPong::K_SLOTS * C::K_BYTES;  // byte offset of the V slots
    constexpr int O_STAGE = V_RING + PingPong::V_SLOTS * C::V_BYTES;   // byte offset of the output staging rows
    static_assert(DV % PingPong::O_HALF_COLUMNS == 0, "output rows leave in halves of 64 columns");
    constexpr int RING = PingPong::RING;
    constexpr int PV_MFMAS = 4 * DBLOCKS;
    constexpr int QK_MFMAS = 2 * KSTEPS;
    constexpr int REQUESTS = C::K_LOADS_PER_WAVE + C::V_LOADS_PER_WAVE;
    static_assert(REQUESTS <= 5, "X issues five tile requests");
    static_assert(PV_MFMAS >= RING, "the fragments read ahead in X must all belong to V");

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int group = wave / 4;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int S = sequence_length;

    const int cluster = blockIdx.x % clusters;
    const int member = blockIdx.x / clusters;
    const int members = gridDim.x / clusters;
    const int cluster_heads = batch_heads / clusters;

    const size_t q_stride = (size_t)query_heads * DQK;
    const size_t o_stride = (size_t)query_heads * DV;
    const unsigned k_stride_bytes = (unsigned)key_value_heads * DQK * 2;
    const unsigned v_stride_bytes = (unsigned)key_value_heads * DV * 2;
    const unsigned lds_base = lds_offset_of(lds);

    // operands of an item
    auto key_base = [&](const ForwardItem& item) {
        const int b = item.batch_head / query_heads;
        const int hk = (item.batch_head % query_heads) / (query_heads / key_value_heads);
        return reinterpret_cast<const unsigned char*>(key + ((size_t)b * S * key_value_heads + hk) * DQK);
    };
    auto value_base = [&](const ForwardItem& item) {
        const int b = item.batch_head / query_heads;
        const int hk = (item.batch_head % query_heads) / (query_heads / key_value_heads);
        return reinterpret_cast<const unsigned char*>(value + ((size_t)b * S * key_value_heads + hk) * DV);
    };
    auto tile_count = [&](const ForwardItem& item) { return (min(S, (item.query_block + 1) * C::BM) - 1) / BN + 1; };

    // One 1 KB piece (index `part` of this wave's share) of the K and V tiles that
    // start at key `key0` of the head at (k_head, v_head): parts below
    // K_LOADS_PER_WAVE belong to K, the rest to V.  Rows past the end of the
    // sequence are clamped to the last one: such keys are invisible to every
    // stored query, the data only has to be finite.
    auto request_part = [&](const unsigned char* k_head, const unsigned char* v_head, int key0, int k_slot,
                            int v_slot, int part) {
        const int row_limit = S - 1 - key0;
        if (part < C::K_LOADS_PER_WAVE) {
            const unsigned char* k_tile = k_head + (size_t)key0 * k_stride_bytes;
            const int load = wave * C::K_LOADS_PER_WAVE + part;
            const int position = 64 * load + lane;
            const int row = position / C::K_CHUNKS;
            const int chunk = (position % C::K_CHUNKS) ^ C::k_swizzle(row);
            const unsigned offset = (unsigned)min(row, row_limit) * k_stride_bytes + 16u * chunk;
            direct_load_16_offset(k_tile, offset, lds_base + k_slot * C::K_BYTES + load * 1024);
        } else {
            const unsigned char* v_tile = v_head + (size_t)key0 * v_stride_bytes;
            const int load = wave * C::V_LOADS_PER_WAVE + (part - C::K_LOADS_PER_WAVE);
            const int position = 64 * load + lane;
            const int row = position / C::V_CHUNKS;
            const int chunk = (position % C::V_CHUNKS) ^ (C::v_flip(row) << 2);
            const unsigned offset = (unsigned)min(row, row_limit) * v_stride_bytes + 16u * chunk;
            direct_load_16_offset(v_tile, offset, lds_base + V_RING + v_slot * C::V_BYTES + load * 1024);
        }
    };

    // Per-lane byte offsets of the fragment reads inside a slot.  K: chunk
    // 2*ks + g of row lq sits at position (2*ks + g) ^ swizzle; the XOR only
    // touches the low bits, so KLOW addresses plus immediates cover all k-steps.
    unsigned k_read[KLOW];
    {
        const int t = g ^ C::k_swizzle(lq);
#pragma unroll
        for (int i = 0; i < KLOW; ++i) k_read[i] = lq * C::K_ROW + 16 * ((2 * i) ^ t);
    }
    unsigned v_read[DBLOCKS];
    {
        const int s16 = lane % 16;
        const int v_row = 4 * g + s16 / 4;
        const int in_group = 32 * ((lane / 16) % 2) + 8 * (s16 % 4);
#pragma unroll
        for (int d = 0; d < DBLOCKS; ++d) v_read[d] = v_row * C::V_ROW + 64 * (d ^ C::v_flip(v_row)) + in_group;
    }
    auto k_fragment = [&](const unsigned char* k_tile, int ks, int mb) -> bf16x8 {
        return *reinterpret_cast<const bf16x8*>(k_tile + k_read[ks % KLOW] + (ks / KLOW) * (SPAN * 16) +
                                                mb * 32 * C::K_ROW);
    };
    auto v_fragment = [&](const unsigned char* v_tile, int n, int d) -> bf16x8 {
        const unsigned char* first = v_tile + v_read[d] + n * 16 * C::V_ROW;
        const s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)first);
        const s16x4 high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((transposing_read_pointer)(first + 8 * C::V_ROW));
        return __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    // fragment i of the Y stream: PV_MFMAS fragments of V (16-key step i / DBLOCKS,
    // column block i % DBLOCKS), then QK_MFMAS fragments of K (k-step, key half)
    auto stream_fragment = [&](const unsigned char* v_tile, const unsigned char* k_tile, int i) -> bf16x8 {
        if (i < PV_MFMAS) {
            return v_fragment(v_tile, i / DBLOCKS, i % DBLOCKS);
        }
        return k_fragment(k_tile, (i - PV_MFMAS) / 2, (i - PV_MFMAS) % 2);
    };

    bf16x8 qf[KSTEPS];
    f32x16 o_acc[DBLOCKS];
    f32x16 s_acc[2];
    bf16x8 pf[4];
    bf16x8 ring[RING];
    float row_max, row_sum;
    const float c = scale * LOG2E;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // Q fragments of an item (B operand: column = query lq, k = 16*ks + 8*g + j)
    auto load_queries = [&](const ForwardItem& item) {
        const int row_index = item.query_block * C::BM + 32 * wave + lq;
        const bool valid = row_index < S;
        const int b = item.batch_head / query_heads;
        const int h = item.batch_head % query_heads;
        const bf16_t* row = query + ((size_t)b * S * query_heads + h) * DQK + (size_t)(valid ? row_index : 0) * q_stride + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            u32x4 bits = {0, 0, 0, 0};
            if (valid) {
                bits = *reinterpret_cast<const u32x4*>(row + 16 * ks);
            }
            qf[ks] = __builtin_bit_cast(bf16x8, bits);
        }
    };

    ForwardItem item, next_item;
    if (!forward_item(0, member, members, cluster, clusters, cluster_heads, query_blocks, item)) {
        return;   // uniform over the workgroup
    }
    bool has_next = forward_item(1, member, members, cluster, clusters, cluster_heads, query_blocks, next_item);

    // ---- prologue of the first item: its queries and its tiles 0 and 1
    load_queries(item);
    wait_vector_memory<0>();
    {
        const unsigned char* k_head = key_base(item);
        const unsigned char* v_head = value_base(item);
#pragma unroll
        for (int part = 0; part < REQUESTS; ++part) request_part(k_head, v_head, 0, 0, 0, part);
#pragma unroll
        for (int part = 0; part < REQUESTS; ++part) request_part(k_head, v_head, BN, 1, 1, part);
    }
    wait_vector_memory<0>();
    workgroup_barrier();

    int k_slot = 0;     // slot of K of the current stream tile (stream index % 3)
    int v_slot = 0;     // slot of V of the current stream tile (stream index % 4)
    int round = 0;
    bool shifted = false;
    while (true) {
        const int tiles = tile_count(item);
        const int wave_q0 = item.query_block * C::BM + 32 * wave;
        const int q_row = wave_q0 + lq;
        const unsigned char* k_head = key_base(item);
        const unsigned char* v_head = value_base(item);
        const unsigned char* next_k_head = has_next ? key_base(next_item) : k_head;
        const unsigned char* next_v_head = has_next ? value_base(next_item) : v_head;

        // S(0) of the item; its K tile was requested two tiles ago
        {
            const unsigned char* k_tile = lds + k_slot * C::K_BYTES;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    s_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_fragment(k_tile, ks, mb), qf[ks],
                                                                        ks == 0 ? zero : s_acc[mb], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[d][i] = 0.f;
        }
        row_max = -INFINITY;
        row_sum = 0.f;
        if (!shifted) {
            shifted = true;
            if (group == 1) {
                workgroup_barrier();
            }
        }

        // X(tile): the requests for stream tile + 2, then the softmax.
        // A wave whose rows all lie before this tile runs it like any other: the
        // mask turns its scores into zeros, and the phases are barrier-locked, so
        // skipping would not end the tile sooner.  (Branching around the
        // arithmetic of such tiles was tried: the extra control flow made the
        // register allocator spill some 200 registers.)
        auto phase_x = [&](int tile) {
            const int key0 = tile * BN;
            const int k_slot2 = k_slot == 0 ? 2 : k_slot - 1;      // (slot + 2) % 3
            const int v_slot2 = (v_slot + 2) & 3;
            const bool from_next = tile + 2 >= tiles;
            const unsigned char* request_k = from_next ? next_k_head : k_head;
            const unsigned char* request_v = from_next ? next_v_head : v_head;
            const int request_key0 = (from_next ? tile + 2 - tiles : tile + 2) * BN;
            auto request_next = [&](int part) {
                if (part < REQUESTS) {
                    request_part(request_k, request_v, request_key0, k_slot2, v_slot2, part);
                }
            };
            // all of this wave's requests first: they have the whole phase and the next to arrive
            request_next(0);
            request_next(1);
            request_next(2);
            request_next(3);
            request_next(4);
            if (key0 + BN - 1 > wave_q0) {  // tile reaches past this wave's first row
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
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                u32x4 packed;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int i = 8 * (n % 2) + 2 * j;
                    const float p0 = __builtin_amdgcn_exp2f(fmaf(s_acc[n / 2][i], c, -offset));
                    const float p1 = __builtin_amdgcn_exp2f(fmaf(s_acc[n / 2][i + 1], c, -offset));
                    row_sum += p0 + p1;   // unrounded: the logsumexp tolerance leaves no room for bf16 sums
                    packed[j] = pack_bf16(p0, p1);
                }
                pf[n] = __builtin_bit_cast(bf16x8, packed);
            }
        };
        // Y(tile): O += V^T P, and with FULL the next S.  The first RING fragments
        // are read before the barrier that separates X from Y.
        auto phase_y = [&](auto full_tag) {
            constexpr bool FULL = decltype(full_tag)::value;
            constexpr int COUNT = FULL ? PV_MFMAS + QK_MFMAS : PV_MFMAS;
            const int k_slot1 = k_slot == 2 ? 0 : k_slot + 1;
            const unsigned char* k_tile = lds + k_slot1 * C::K_BYTES;           // K(tile + 1)
            const unsigned char* v_tile = lds + V_RING + v_slot * C::V_BYTES;   // V(tile)
#pragma unroll
            for (int i = 0; i < RING; ++i) ring[i] = stream_fragment(v_tile, k_tile, i);
            workgroup_barrier();
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int i = 0; i < COUNT; ++i) {
                if (i < PV_MFMAS) {
                    o_acc[i % DBLOCKS] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % RING], pf[i / DBLOCKS],
                                                                                 o_acc[i % DBLOCKS], 0, 0, 0);
                } else {
                    const int ks = (i - PV_MFMAS) / 2;
                    const int mb = (i - PV_MFMAS) % 2;
                    s_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % RING], qf[ks],
                                                                        ks == 0 ? zero : s_acc[mb], 0, 0, 0);
                }
                if (i + RING < COUNT) {
                    ring[i % RING] = stream_fragment(v_tile, k_tile, i + RING);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
            wait_vector_memory<0>();   // this wave's requests of X(tile)
            workgroup_barrier();
            k_slot = k_slot1;
            v_slot = (v_slot + 1) & 3;
        };

        for (int tile = 0; tile + 1 < tiles; ++tile) {
            phase_x(tile);
            phase_y(std::true_type{});
        }
        // Last tile: its scores exist already, so the query registers are free: the next item's queries load
        // while this tile finishes.
        if (has_next) {
            load_queries(next_item);
        }
        phase_x(tiles - 1);
        phase_y(std::false_type{});

        // ---- epilogue: normalise, round, and store rows and logsumexp.  A lane holds, per column block, four
        // runs of four columns of one query; the rows go through this wave's staging rows in LDS, 64 columns
        // at a time, so that every store instruction writes eight whole 128-byte lines.  Only this wave touches
        // its staging rows; the two groups come through here in different phases and share them.
        {
            const int fresh = fresh_lane_id();   // nothing of the address arithmetic below is carried through the tile loop
            const int row = fresh % 32;
            const int half_wave = fresh / 32;
            const float total = half_wave_sum(row_sum);
            const float inverse = 1.0f / total;
            const int b = item.batch_head / query_heads;
            const int h = item.batch_head % query_heads;
            if (half_wave == 0 && wave_q0 + row < S) {
                logsumexp[((size_t)b * query_heads + h) * S + wave_q0 + row] = row_max * scale + __logf(total);
            }
            bf16_t* o_head = output + ((size_t)b * S * query_heads + h) * DV;
            unsigned char* o_lds = lds + O_STAGE + (wave % 4) * PingPong::O_WAVE_BYTES;
            constexpr int HALVES = DV / PingPong::O_HALF_COLUMNS;
            constexpr int HALF_BLOCKS = PingPong::O_HALF_COLUMNS / 32;
#pragma unroll
            for (int half = 0; half < HALVES; ++half) {
#pragma unroll
                for (int db = 0; db < HALF_BLOCKS; ++db) {
                    const int d = half * HALF_BLOCKS + db;
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) {
                        u32x2 packed;
                        packed.x = pack_bf16(o_acc[d][4 * i4 + 0] * inverse, o_acc[d][4 * i4 + 1] * inverse);
                        packed.y = pack_bf16(o_acc[d][4 * i4 + 2] * inverse, o_acc[d][4 * i4 + 3] * inverse);
                        *reinterpret_cast<u32x2*>(o_lds + row * PingPong::O_PITCH + 2 * (32 * db + 8 * i4 + 4 * half_wave)) = packed;
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
                __builtin_amdgcn_wave_barrier();
                // 32 rows x 128 bytes: eight lanes per row, eight rows per pass
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
                    const int r = 8 * pass + fresh / 8;
                    const u32x4 bits = *reinterpret_cast<const u32x4*>(o_lds + r * PingPong::O_PITCH + 16 * (fresh % 8));
                    if (wave_q0 + r < S) {
                        *reinterpret_cast<u32x4*>(o_head + (size_t)(wave_q0 + r) * o_stride +
                                                  half * PingPong::O_HALF_COLUMNS + 8 * (fresh % 8)) = bits;
                    }
                }
                __builtin_amdgcn_wave_barrier();   // the reads above precede the next half's writes
            }
        }
        if (!has_next) {
            break;
        }
        item = next_item;
        ++round;
        has_next = forward_item(round + 1, member, members, cluster, clusters, cluster_heads, query_blocks, next_item);
    }
    if (group == 0) {
        workgroup_barrier();
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
    // per-lane byte offsets inside a key tile are 32-bit
    if ((long long)key_value_heads * (DQK > DV ? DQK : DV) * 2 * C::BN > 0x7fffffffLL) {
        throw std::invalid_argument("attention forward: key_value_heads * head size is too large");
    }
    auto kernel = attention_forward_kernel<DQK, DV, NWAVES>;
    if (C::LDS_BYTES > 64 * 1024) {
        static hip_common::OncePerDevice raised;
        raised.run([&] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES));
        });
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(C::THREADS), C::LDS_BYTES, stream, output, logsumexp, query,
                       key, value, sequence_length, query_heads, key_value_heads, query_blocks, scale);
    HIP_CHECK(hipGetLastError());
}

template <int DQK, int DV>
void launch_forward_pingpong(bf16_t* output, float* logsumexp, const bf16_t* query, const bf16_t* key,
                             const bf16_t* value, int batch_size, int sequence_length, int query_heads,
                             int key_value_heads, float scale, hipStream_t stream) {
    using C = FwdConfig<DQK, DV, 8>;
    constexpr int LDS_BYTES = PingPong::K_SLOTS * C::K_BYTES + PingPong::V_SLOTS * C::V_BYTES + PingPong::O_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "the tile slots and the output staging rows must fit the LDS");
    const int query_blocks = (sequence_length + C::BM - 1) / C::BM;
    const long long batch_heads = (long long)batch_size * query_heads;
    if (batch_heads * query_blocks > 0x7fffffffLL) {
        throw std::invalid_argument("attention forward: batch*heads*query_blocks exceeds the item limit");
    }
    if ((long long)key_value_heads * (DQK > DV ? DQK : DV) * 2 * C::BN > 0x7fffffffLL) {
        throw std::invalid_argument("attention forward: key_value_heads * head size is too large");
    }
    // one workgroup per compute unit (the LDS footprint admits no second one)
    const int compute_units = hip_common::compute_units_of_current_device();
    const int clusters = (batch_heads % PingPong::CLUSTERS == 0 && compute_units >= PingPong::CLUSTERS)
                             ? PingPong::CLUSTERS : 1;
    long long grid = compute_units / clusters * clusters;
    const long long items_per_cluster = batch_heads / clusters * query_blocks;
    if (grid / clusters > items_per_cluster) {
        grid = items_per_cluster * clusters;
    }
    auto kernel = attention_forward_pingpong_kernel<DQK, DV>;
    static hip_common::OncePerDevice raised;
    raised.run([&] {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
    });
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(C::THREADS), LDS_BYTES, stream, output, logsumexp, query,
                       key, value, sequence_length, query_heads, key_value_heads, query_blocks, (int)batch_heads,
                       clusters, scale);
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
    // the persistent kernel streams two tiles ahead across items: every item needs two tiles
    const bool large = rows >= 256LL * 256 * 2 && sequence_length >= 128;
#define DSCUDA_FWD_CASE(DQK, DV)                                                                                  \
    if (qk_head_size == DQK && v_head_size == DV) {                                                               \
        if constexpr (DV >= 128) {                                                                                \
            if (large) {                                                                                          \
                launch_forward_pingpong<DQK, DV>(output, logsumexp, query, key, value, batch_size,               \
                                                 sequence_length, query_heads, key_value_heads, scale, stream);   \
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
