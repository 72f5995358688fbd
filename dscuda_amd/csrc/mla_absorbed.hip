// Absorbed-query MLA backward for gfx950 (C = 512 latent + R = 64 rope, one
// shared KV head).  Takes the place of the reference's
// mla_query_backward_kernel and mla_kv_backward_kernel
// (kernels/attention/mla/sm89.cu:295-411) and keeps their contract: the four
// gradients are overwritten, each gradient row has exactly one writer (no
// atomics, deterministic), no workspace.  The mathematics is
// reference/python/mla.py:42-57:
//     P = exp(S - LSE),  dP = dO latent^T,  delta = sum(dO * O),
//     dS = P (dP - delta) scale,
//     dQ = dS [latent|rope],  d[latent|rope] = dS^T [q_lat|q_rope],  dlatent += P^T dO.
//
// "Rows" are the (token, head) pairs of one batch element in memory order
// (row = token*H + head), which makes query / dO / O rows contiguous 512- and
// 64-wide vectors.  Both kernels run every product on bf16 MFMA 32x32x16 with
// fp32 accumulation and keep all operands in LDS, 32 rows or keys at a time,
// each tile stored row-major and (where it is also needed with its row index
// as the contraction index) transposed, as in the per-head backward.
//
//   query gradients   a workgroup owns 32 rows and walks the keys up to the
//                     last token of those rows.  Every wave forms the 32x32
//                     S^T and dP^T of the tile, and accumulates dQ^T for its
//                     own share of the 18 column blocks.
//   key gradients     a workgroup owns 32 keys (held in registers) and walks
//                     the rows from the first token that can see them.  Every
//                     wave forms S and dP of the tile and accumulates its
//                     own four latent column blocks (key path and value path
//                     in the same accumulator) plus a rope column block.
//
// The score products are repeated by the four waves of a workgroup; this entry
// point is kept for interface parity and correctness at the reference's
// shapes, the throughput path of this library is the per-head form.
#include "attn_kernels.h"
#include "hip_common.h"

#include <stdexcept>
#include <string>

namespace dscuda {
namespace {

constexpr int RANK = 512;
constexpr int ROPE = 64;
constexpr int WIDTH = RANK + ROPE;
constexpr int TILE = 32;
constexpr int THREADS = 256;

template <int D>
struct Tile32 {
    static constexpr int PITCH = 2 * D + 16;                // row-major copy
    static constexpr int NATURAL_BYTES = TILE * PITCH;
    static constexpr int T_PITCH = 2 * TILE;                 // transposed copy: 64-byte rows
    static constexpr int TRANSPOSED_BYTES = D * T_PITCH;
    static constexpr int UNITS = (TILE / 4) * (D / 4);       // 4 rows x 4 columns
    static constexpr int PER_THREAD = (UNITS + THREADS - 1) / THREADS;
};

// Stage a [32][D] tile whose row `row` starts at row_pointer(row) (nullptr: zero
// row) into LDS, row-major and/or transposed.  Columns [column0, column0 + D_PART)
// of the LDS tile come from this call, so a tile can be assembled from two tensors.
template <int D, int D_PART, bool NATURAL, bool TRANSPOSED, typename RowPointer>
__device__ __forceinline__ void stage_tile(unsigned char* natural, unsigned char* transposed, int column0,
                                           RowPointer row_pointer, int tid) {
    using T = Tile32<D>;
    constexpr int UNITS = (TILE / 4) * (D_PART / 4);
    for (int unit = tid; unit < UNITS; unit += THREADS) {
        const int c4 = unit % (D_PART / 4);
        const int rg = unit / (D_PART / 4);
        u32x2 r[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bf16_t* source = row_pointer(4 * rg + j);
            r[j] = u32x2{0, 0};
            if (source != nullptr) r[j] = *reinterpret_cast<const u32x2*>(source + 4 * c4);
        }
        const int column = column0 + 4 * c4;
        if (NATURAL) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                *reinterpret_cast<u32x2*>(natural + (4 * rg + j) * T::PITCH + 2 * column) = r[j];
            }
        }
        if (TRANSPOSED) {
            // rows 4*rg .. +3 = 16*n + 8*a + 4*g' + (0..3)  ->  position 16*n + 8*g' + 4*a
            const int n = rg / 4;
            const int a = (rg % 4) / 2;
            const int gp = rg % 2;
            const int chunk = 2 * n + gp;
            u32x2 t[4];
            t[0] = u32x2{(r[0].x & 0xffffu) | (r[1].x << 16), (r[2].x & 0xffffu) | (r[3].x << 16)};
            t[1] = u32x2{(r[0].x >> 16) | (r[1].x & 0xffff0000u), (r[2].x >> 16) | (r[3].x & 0xffff0000u)};
            t[2] = u32x2{(r[0].y & 0xffffu) | (r[1].y << 16), (r[2].y & 0xffffu) | (r[3].y << 16)};
            t[3] = u32x2{(r[0].y >> 16) | (r[1].y & 0xffff0000u), (r[2].y >> 16) | (r[3].y & 0xffff0000u)};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = column + e;
                const int swz = chunk ^ ((col >> 2) & 3);
                *reinterpret_cast<u32x2*>(transposed + col * T::T_PITCH + 16 * swz + 8 * a) = t[e];
            }
        }
    }
}

template <int D>
__device__ __forceinline__ bf16x8 natural_fragment(const unsigned char* natural, int row, int ks, int g) {
    return *reinterpret_cast<const bf16x8*>(natural + row * Tile32<D>::PITCH + 32 * ks + 16 * g);
}

// column `column`, tile rows {16n + 4g .. +3, 16n + 8 + 4g .. +3}
template <int D>
__device__ __forceinline__ bf16x8 transposed_fragment(const unsigned char* transposed, int column, int n, int g) {
    const int swz = (2 * n + g) ^ ((column >> 2) & 3);
    return *reinterpret_cast<const bf16x8*>(transposed + column * Tile32<D>::T_PITCH + 16 * swz);
}

__device__ __forceinline__ void clear(f32x16& value) {
#pragma unroll
    for (int i = 0; i < 16; ++i) value[i] = 0.f;
}

// Per-row statistics of a 32-row tile: lse*log2e, delta = sum(dO*O), token index.
// Eight threads share a row and 64 columns each.
__device__ __forceinline__ void stage_row_statistics(float* lse2, float* delta, int* token_of, const bf16_t* dout_rows,
                                                     const bf16_t* out_rows, const float* lse_batch, long long row0,
                                                     long long rows, int heads, int sequence_length, int tid) {
    const int local = tid / 8;
    const int part = tid % 8;
    const long long row = row0 + local;
    float sum = 0.f;
    if (row < rows) {
        const bf16_t* a_row = dout_rows + row * RANK + 64 * part;
        const bf16_t* b_row = out_rows + row * RANK + 64 * part;
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(a_row + 8 * v);
            const u32x4 b = *reinterpret_cast<const u32x4*>(b_row + 8 * v);
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
    if (part == 0) {
        if (row < rows) {
            const int token = (int)(row / heads);
            const int head = (int)(row % heads);
            lse2[local] = lse_batch[(size_t)head * sequence_length + token] * LOG2E;
            delta[local] = sum;
            token_of[local] = token;
        } else {
            lse2[local] = 0.f;
            delta[local] = 0.f;
            token_of[local] = -1;   // sees no key
        }
    }
}

// ---- query gradients -----------------------------------------------------------

struct QueryGradLayout {
    static constexpr int Q_ROWS = 0;                                          // [32][576] row-major
    static constexpr int DO_ROWS = Q_ROWS + Tile32<WIDTH>::NATURAL_BYTES;     // [32][512] row-major
    static constexpr int K_NATURAL = DO_ROWS + Tile32<RANK>::NATURAL_BYTES;   // [32 keys][576]
    static constexpr int K_TRANSPOSED = K_NATURAL + Tile32<WIDTH>::NATURAL_BYTES;
    static constexpr int STATS = K_TRANSPOSED + Tile32<WIDTH>::TRANSPOSED_BYTES;
    static constexpr int LDS_BYTES = STATS + 3 * TILE * 4;
};

__global__ __launch_bounds__(THREADS) void mla_absorbed_query_gradient_kernel(
    bf16_t* __restrict__ query_latent_gradient, bf16_t* __restrict__ query_rope_gradient,
    const bf16_t* __restrict__ output_gradient, const bf16_t* __restrict__ output, const float* __restrict__ logsumexp,
    const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int sequence_length, int heads,
    int row_blocks, float scale) {
    using L = QueryGradLayout;
    constexpr int BLOCKS = WIDTH / 32;                 // 18 column blocks of dQ
    constexpr int OWN = (BLOCKS + 3) / 4;              // at most 5 per wave

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    unsigned char* q_rows = lds + L::Q_ROWS;
    unsigned char* do_rows = lds + L::DO_ROWS;
    unsigned char* k_natural = lds + L::K_NATURAL;
    unsigned char* k_transposed = lds + L::K_TRANSPOSED;
    float* lse2 = reinterpret_cast<float*>(lds + L::STATS);
    float* delta = lse2 + TILE;
    int* token_of = reinterpret_cast<int*>(delta + TILE);

    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int T = sequence_length;

    const int batch = blockIdx.x / row_blocks;
    const int row_block = row_blocks - 1 - blockIdx.x % row_blocks;   // latest rows (most keys) first
    const long long rows = (long long)T * heads;
    const long long row0 = (long long)row_block * TILE;
    const long long batch_row0 = (long long)batch * rows;

    const bf16_t* ql = query_latent + batch_row0 * RANK;
    const bf16_t* qr = query_rope + batch_row0 * ROPE;
    const bf16_t* dout = output_gradient + batch_row0 * RANK;
    const bf16_t* out = output + batch_row0 * RANK;
    const bf16_t* latent = kv_latent + (size_t)batch * T * RANK;
    const bf16_t* rope = key_rope + (size_t)batch * T * ROPE;

    stage_tile<WIDTH, RANK, true, false>(q_rows, nullptr, 0, [&](int r) -> const bf16_t* {
        return row0 + r < rows ? ql + (row0 + r) * RANK : nullptr; }, tid);
    stage_tile<WIDTH, ROPE, true, false>(q_rows, nullptr, RANK, [&](int r) -> const bf16_t* {
        return row0 + r < rows ? qr + (row0 + r) * ROPE : nullptr; }, tid);
    stage_tile<RANK, RANK, true, false>(do_rows, nullptr, 0, [&](int r) -> const bf16_t* {
        return row0 + r < rows ? dout + (row0 + r) * RANK : nullptr; }, tid);
    stage_row_statistics(lse2, delta, token_of, dout, out, logsumexp + (size_t)batch * heads * T, row0, rows, heads, T,
                         tid);
    __syncthreads();

    const float row_lse2 = lse2[lq];
    const float row_delta = delta[lq];
    const int row_token = token_of[lq];
    const long long last_row = min(rows, row0 + TILE) - 1;
    const int visible = (int)(last_row / heads) + 1;
    const int tiles = (visible + TILE - 1) / TILE;
    const float c = scale * LOG2E;

    f32x16 dq_acc[OWN];
#pragma unroll
    for (int j = 0; j < OWN; ++j) clear(dq_acc[j]);

    for (int tile = 0; tile < tiles; ++tile) {
        const int key0 = tile * TILE;
        __syncthreads();
        stage_tile<WIDTH, RANK, true, true>(k_natural, k_transposed, 0, [&](int r) -> const bf16_t* {
            return key0 + r < T ? latent + (size_t)(key0 + r) * RANK : nullptr; }, tid);
        stage_tile<WIDTH, ROPE, true, true>(k_natural, k_transposed, RANK, [&](int r) -> const bf16_t* {
            return key0 + r < T ? rope + (size_t)(key0 + r) * ROPE : nullptr; }, tid);
        __syncthreads();

        f32x16 s_acc, dp_acc;   // (keys x rows): lane holds row lq and keys key0 + 8*(i/4) + 4*g + i%4
        clear(s_acc);
        clear(dp_acc);
#pragma unroll 4
        for (int ks = 0; ks < WIDTH / 16; ++ks) {
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(natural_fragment<WIDTH>(k_natural, lq, ks, g),
                                                            natural_fragment<WIDTH>(q_rows, lq, ks, g), s_acc, 0, 0, 0);
        }
#pragma unroll 4
        for (int ks = 0; ks < RANK / 16; ++ks) {
            dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(natural_fragment<WIDTH>(k_natural, lq, ks, g),
                                                             natural_fragment<RANK>(do_rows, lq, ks, g), dp_acc, 0, 0, 0);
        }
        bf16x8 dsf[2];
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            u32x4 packed;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float ds[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int i = 8 * n + 2 * j + e;
                    const int k = key0 + 8 * (i / 4) + 4 * g + i % 4;
                    float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[i], c, -row_lse2));
                    if (k > row_token) probability = 0.f;
                    ds[e] = probability * (dp_acc[i] - row_delta) * scale;
                }
                packed[j] = pack_bf16(ds[0], ds[1]);
            }
            dsf[n] = __builtin_bit_cast(bf16x8, packed);
        }
#pragma unroll
        for (int j = 0; j < OWN; ++j) {
            const int block = min(wave + 4 * j, BLOCKS - 1);   // the clamped duplicate is never stored
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                dq_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    transposed_fragment<WIDTH>(k_transposed, 32 * block + lq, n, g), dsf[n], dq_acc[j], 0, 0, 0);
            }
        }
    }

    // lane holds row lq and columns 32*block + 8*(i/4) + 4*g + i%4
    const long long row = row0 + lq;
    if (row < rows) {
#pragma unroll
        for (int j = 0; j < OWN; ++j) {
            const int block = wave + 4 * j;
            if (block < BLOCKS) {
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    u32x2 packed;
                    packed.x = pack_bf16(dq_acc[j][4 * i4 + 0], dq_acc[j][4 * i4 + 1]);
                    packed.y = pack_bf16(dq_acc[j][4 * i4 + 2], dq_acc[j][4 * i4 + 3]);
                    const int column = 32 * block + 8 * i4 + 4 * g;
                    bf16_t* destination = column < RANK
                        ? query_latent_gradient + (batch_row0 + row) * RANK + column
                        : query_rope_gradient + (batch_row0 + row) * ROPE + (column - RANK);
                    *reinterpret_cast<u32x2*>(destination) = packed;
                }
            }
        }
    }
}

// ---- key gradients -------------------------------------------------------------

struct KeyGradLayout {
    static constexpr int Q_NATURAL = 0;                                            // [32 rows][576]
    static constexpr int Q_TRANSPOSED = Q_NATURAL + Tile32<WIDTH>::NATURAL_BYTES;  // [576][32 rows]
    static constexpr int DO_NATURAL = Q_TRANSPOSED + Tile32<WIDTH>::TRANSPOSED_BYTES;
    static constexpr int DO_TRANSPOSED = DO_NATURAL + Tile32<RANK>::NATURAL_BYTES;
    static constexpr int STATS = DO_TRANSPOSED + Tile32<RANK>::TRANSPOSED_BYTES;
    static constexpr int LDS_BYTES = STATS + 3 * TILE * 4;
};

__global__ __launch_bounds__(THREADS) void mla_absorbed_key_gradient_kernel(
    bf16_t* __restrict__ kv_latent_gradient, bf16_t* __restrict__ key_rope_gradient,
    const bf16_t* __restrict__ output_gradient, const bf16_t* __restrict__ output, const float* __restrict__ logsumexp,
    const bf16_t* __restrict__ query_latent, const bf16_t* __restrict__ query_rope,
    const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope, int sequence_length, int heads,
    int key_blocks, float scale) {
    using L = KeyGradLayout;
    constexpr int QK_STEPS = WIDTH / 16;   // 36
    constexpr int V_STEPS = RANK / 16;     // 32

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    unsigned char* q_natural = lds + L::Q_NATURAL;
    unsigned char* q_transposed = lds + L::Q_TRANSPOSED;
    unsigned char* do_natural = lds + L::DO_NATURAL;
    unsigned char* do_transposed = lds + L::DO_TRANSPOSED;
    float* lse2 = reinterpret_cast<float*>(lds + L::STATS);
    float* delta = lse2 + TILE;
    int* token_of = reinterpret_cast<int*>(delta + TILE);

    const int tid = threadIdx.x;
    const int wave = tid / 64;
    const int lane = tid % 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int T = sequence_length;

    const int batch = blockIdx.x / key_blocks;
    const int key_block = blockIdx.x % key_blocks;   // key block 0 is seen by every row: heaviest first
    const int k0 = key_block * TILE;
    const int key = k0 + lq;
    const long long rows = (long long)T * heads;
    const long long batch_row0 = (long long)batch * rows;

    const bf16_t* ql = query_latent + batch_row0 * RANK;
    const bf16_t* qr = query_rope + batch_row0 * ROPE;
    const bf16_t* dout = output_gradient + batch_row0 * RANK;
    const bf16_t* out = output + batch_row0 * RANK;
    const bf16_t* latent = kv_latent + (size_t)batch * T * RANK;
    const bf16_t* rope = key_rope + (size_t)batch * T * ROPE;

    // this workgroup's keys as B operands (column = key lq); the value operand is the latent part
    bf16x8 kf[QK_STEPS];
    {
        const bool valid = key < T;
        const size_t k = valid ? key : 0;
#pragma unroll
        for (int ks = 0; ks < QK_STEPS; ++ks) {
            u32x4 bits = {0, 0, 0, 0};
            if (valid) {
                const bf16_t* source = ks < V_STEPS ? latent + k * RANK + 16 * ks + 8 * g
                                                    : rope + k * ROPE + 16 * (ks - V_STEPS) + 8 * g;
                bits = *reinterpret_cast<const u32x4*>(source);
            }
            kf[ks] = __builtin_bit_cast(bf16x8, bits);
        }
    }

    f32x16 latent_acc[4], rope_acc;   // column blocks 4*wave + j of the latent, block wave%2 of the rope part
#pragma unroll
    for (int j = 0; j < 4; ++j) clear(latent_acc[j]);
    clear(rope_acc);

    const float c = scale * LOG2E;
    const long long first_row = (long long)k0 * heads;             // first row that can see key k0
    const int first_tile = (int)(first_row / TILE);
    const int last_tile = (int)((rows - 1) / TILE);

    for (int tile = first_tile; tile <= last_tile; ++tile) {
        const long long row0 = (long long)tile * TILE;
        __syncthreads();
        stage_tile<WIDTH, RANK, true, true>(q_natural, q_transposed, 0, [&](int r) -> const bf16_t* {
            return row0 + r < rows ? ql + (row0 + r) * RANK : nullptr; }, tid);
        stage_tile<WIDTH, ROPE, true, true>(q_natural, q_transposed, RANK, [&](int r) -> const bf16_t* {
            return row0 + r < rows ? qr + (row0 + r) * ROPE : nullptr; }, tid);
        stage_tile<RANK, RANK, true, true>(do_natural, do_transposed, 0, [&](int r) -> const bf16_t* {
            return row0 + r < rows ? dout + (row0 + r) * RANK : nullptr; }, tid);
        stage_row_statistics(lse2, delta, token_of, dout, out, logsumexp + (size_t)batch * heads * T, row0, rows, heads,
                             T, tid);
        __syncthreads();

        f32x16 s_acc, dp_acc;   // (rows x keys): lane holds key lq and tile rows 8*(i/4) + 4*g + i%4
        clear(s_acc);
        clear(dp_acc);
#pragma unroll
        for (int ks = 0; ks < QK_STEPS; ++ks) {
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(natural_fragment<WIDTH>(q_natural, lq, ks, g), kf[ks], s_acc,
                                                            0, 0, 0);
        }
#pragma unroll
        for (int ks = 0; ks < V_STEPS; ++ks) {
            dp_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(natural_fragment<RANK>(do_natural, lq, ks, g), kf[ks],
                                                             dp_acc, 0, 0, 0);
        }
        bf16x8 pf[2], dsf[2];
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            u32x4 p_packed, ds_packed;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int i4 = 2 * n + half;
                const int local = 8 * i4 + 4 * g;
                const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse2 + local);
                const f32x4 delta4 = *reinterpret_cast<const f32x4*>(delta + local);
                const u32x4 token4 = *reinterpret_cast<const u32x4*>(token_of + local);
                float p[4], ds[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 4 * i4 + e;
                    float probability = __builtin_amdgcn_exp2f(fmaf(s_acc[i], c, -lse4[e]));
                    if (key > (int)token4[e]) probability = 0.f;
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
#pragma unroll
        for (int n = 0; n < 2; ++n) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int column = 32 * (4 * wave + j) + lq;
                latent_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    dsf[n], transposed_fragment<WIDTH>(q_transposed, column, n, g), latent_acc[j], 0, 0, 0);
                latent_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    pf[n], transposed_fragment<RANK>(do_transposed, column, n, g), latent_acc[j], 0, 0, 0);
            }
            rope_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                dsf[n], transposed_fragment<WIDTH>(q_transposed, RANK + 32 * (wave % 2) + lq, n, g), rope_acc, 0, 0, 0);
        }
    }

    // lane holds column (block, lq) and keys k0 + 8*(i/4) + 4*g + i%4
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int k = k0 + 8 * (i / 4) + 4 * g + i % 4;
        if (k < T) {
            __bf16* latent_row = reinterpret_cast<__bf16*>(kv_latent_gradient) + ((size_t)batch * T + k) * RANK;
#pragma unroll
            for (int j = 0; j < 4; ++j) latent_row[32 * (4 * wave + j) + lq] = (__bf16)latent_acc[j][i];
            if (wave < 2) {
                __bf16* rope_row = reinterpret_cast<__bf16*>(key_rope_gradient) + ((size_t)batch * T + k) * ROPE;
                rope_row[32 * wave + lq] = (__bf16)rope_acc[i];
            }
        }
    }
}

template <typename Kernel>
void raise_lds_limit(Kernel kernel, int bytes) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  bytes));
}

}  // namespace

void mla_absorbed_backward_dispatch(bf16_t* query_latent_gradient, bf16_t* query_rope_gradient,
                                    bf16_t* kv_latent_gradient, bf16_t* key_rope_gradient,
                                    const bf16_t* output_gradient, const bf16_t* output, const float* logsumexp,
                                    const bf16_t* query_latent, const bf16_t* query_rope, const bf16_t* kv_latent,
                                    const bf16_t* key_rope, int batch_size, int sequence_length, int heads, float scale,
                                    hipStream_t stream) {
    static thread_local bool prepared = false;
    if (!prepared) {
        raise_lds_limit(mla_absorbed_query_gradient_kernel, QueryGradLayout::LDS_BYTES);
        raise_lds_limit(mla_absorbed_key_gradient_kernel, KeyGradLayout::LDS_BYTES);
        prepared = true;
    }
    const long long rows = (long long)sequence_length * heads;
    const long long row_blocks = (rows + TILE - 1) / TILE;
    const long long key_blocks = (sequence_length + TILE - 1) / TILE;
    if (row_blocks * batch_size > 0x7fffffffLL) {
        throw std::invalid_argument("MLA backward: batch*tokens*heads exceeds the grid limit");
    }
    hipLaunchKernelGGL(mla_absorbed_query_gradient_kernel, dim3((unsigned)(row_blocks * batch_size)), dim3(THREADS),
                       QueryGradLayout::LDS_BYTES, stream, query_latent_gradient, query_rope_gradient, output_gradient,
                       output, logsumexp, query_latent, query_rope, kv_latent, key_rope, sequence_length, heads,
                       (int)row_blocks, scale);
    HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(mla_absorbed_key_gradient_kernel, dim3((unsigned)(key_blocks * batch_size)), dim3(THREADS),
                       KeyGradLayout::LDS_BYTES, stream, kv_latent_gradient, key_rope_gradient, output_gradient, output,
                       logsumexp, query_latent, query_rope, kv_latent, key_rope, sequence_length, heads,
                       (int)key_blocks, scale);
    HIP_CHECK(hipGetLastError());
}

}  // namespace dscuda
