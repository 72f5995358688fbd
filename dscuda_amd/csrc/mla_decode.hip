// Absorbed-weight MLA over a shared 512+64 latent KV stream for gfx950:
// single-token decode from a paged cache (split-KV + merge) and the causal
// absorbed prefill forward.  Takes the place of the reference's
// mla_decode_split_kernel / mla_decode_combine_kernel
// (kernels/attention/mla/sm89.cu:413-507) and mla_forward_kernel (:156-291);
// the decomposition below is built around 64-lane MFMA waves and the 160 KB
// LDS and shares nothing with their per-head scalar loops.
//
// Rows and units
//   A workgroup (4 waves) owns 128 "rows" -- the heads of one sequence in
//   decode, consecutive (token, head) pairs in prefill -- and walks the key
//   stream in units of 32 tokens.  Every row of a workgroup reads the same
//   keys, so a 36 KB unit is fetched from HBM once and feeds 128 rows x
//   (576 + 512) x 2 flop per token: the only way the 242 flop/byte of the
//   H = 128 decode stays on the HBM roofline.  Each wave owns 32 rows: the
//   scores are produced transposed, S^T (32 keys x 32 rows) = K_unit Q^T with
//   Q held in registers (36 k-steps), and O^T (512 x 32 rows) += V^T P^T is
//   accumulated in 256 accumulator registers per lane.
//
// One LDS copy serves K and V
//   V is the first 512 columns of the same rows.  A unit is stored once,
//   row-major, and read two ways: 16-byte row reads for the K operand, and
//   ds_read_b64_tr_b16 (a 4 keys x 16 columns block transposed across 16
//   lanes) for the V^T operand.  A ring of four 36 KB slots holds the stream.
//
// Global -> LDS without registers
//   Units arrive by global_load_lds (16 bytes per lane, a wave instruction
//   fills 1 KB of consecutive LDS).  With no padding possible inside that 1 KB
//   the bank spread comes from a swizzle applied on the global side: the
//   16-byte chunk c of row r lives at slot 72*r + (c ^ f(r)), f(r) = the three
//   bits of r>>1 with bits 0 and 2 exchanged.  That makes both the 16-row
//   column reads (K operand) and the 4-row x 64-byte block reads (V operand)
//   conflict free, and every LDS address of the inner loops stays a per-lane
//   base plus an immediate.
//
// Scheduling (decode)
//   The 64-token tiles of all sequences form one list that is cut into equal ranges,
//   one per workgroup (one workgroup per CU), so uneven lengths balance to
//   within a tile.  The cut is a small table (the plan) that a one-workgroup
//   kernel derives from the lengths on the device, so the call stays
//   capturable; a caller that decodes several layers over the same lengths
//   builds it once and passes it in.  A range may start or end inside a
//   sequence; such a segment leaves (exponent reference, sum, unnormalised O
//   as bf16) in the caller's workspace at slot workgroup + sequence -- unique
//   because ranges and sequences both advance monotonically -- and a second
//   kernel, spread over the whole chip, merges the slots of a sequence.
//   (Merging inside the first kernel, by the workgroup that delivers the last
//   part of a sequence, was measured: the 64 mergers run alone at the end with
//   one compute unit each, which cost 110 us against 6 for the second kernel.)
//   Sequences that fall inside one range are finished in place.
#include "attn_kernels.h"
#include "hip_common.h"
#include "index_math.h"

#include <algorithm>
#include <cstdint>
#include <stdexcept>
#include <string>

namespace dscuda {
namespace {

constexpr int RANK = 512;
constexpr int ROPE = 64;
constexpr int WIDTH = RANK + ROPE;
constexpr int BN = 64;                      // keys per tile, the grain of the decode work list
constexpr int ROWS = 128;                   // rows per workgroup
constexpr int THREADS = 256;
constexpr int CHUNKS = WIDTH / 8;           // 72 16-byte chunks per key row
constexpr int ROW_BYTES = CHUNKS * 16;      // 1152
constexpr int KSTEPS = WIDTH / 16;          // 36
constexpr int DBLOCKS = RANK / 32;          // 16
constexpr int EPILOGUE_PITCH = 1024 + 16;   // bytes per staged output row

typedef const __attribute__((address_space(1))) void* global_pointer;

__device__ __forceinline__ int swizzle_of_row(int row) {
    return index_math::tile_swizzle<ROW_BYTES>(row);
}

__device__ __forceinline__ float uniform(float value) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, value)));
}

struct KeyStream {
    const bf16_t* latent;      // token t at latent + t*latent_stride, 512 wide
    const bf16_t* rope;        // token t at rope + t*rope_stride, 64 wide
    size_t latent_stride;
    size_t rope_stride;
    const int* block_table;    // nullptr: tokens are stored contiguously
    int page_size;
};

// Score-chain MFMAs with the accumulator held in ordinary vector registers.
// The compiler's own MFMAs take accumulator-file destinations in a kernel this
// large, and that file is fully occupied by the output accumulators.  Issued
// as asm, the hazard bookkeeping is done here.  The first MFMA of a chain starts
// from the inline constant 0 (its destination may not share registers with its
// operands); a dependent MFMA that accumulates into the registers it reads is
// interlocked by hardware; the last MFMA of a chain carries, inside the same
// asm statement, the wait states a vector-ALU reader of the result needs after
// an 8-pass MFMA.
//
// What the hardware does not interlock is a vector-ALU access to the
// accumulator between two MFMAs of a chain, and to the compiler the accumulator
// is an ordinary value after every statement: nothing in the language stops it
// from moving the value to other registers right there (it has done so, to
// place the tail of a chain where a later copy wanted it -- the moves read a
// result the matrix pipeline had not written yet).  Two things keep that from
// happening unnoticed: the code below never copies a chain's accumulator in
// C++ (move_scores is asm as well), and tests/test_decode_isa.py reads the
// generated ISA of every kernel in this file and fails if any instruction
// other than the chain's own MFMAs touches an accumulator's registers before
// the wait states have passed.
__device__ __forceinline__ void score_mfma_first(f32x16& accumulator, const bf16x8& a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(accumulator) : "v"(a), "v"(b));
}

__device__ __forceinline__ void score_mfma(f32x16& accumulator, const bf16x8& a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(accumulator) : "v"(a), "v"(b));
}

__device__ __forceinline__ void score_mfma_last(f32x16& accumulator, const bf16x8& a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 7" : "+v"(accumulator) : "v"(a), "v"(b));
}

// target = source, as one opaque statement: the compiler can neither fold it into the
// chain that produced `source` nor start it early.
__device__ __forceinline__ void move_scores(f32x16& target, const f32x16& source) {
    typedef unsigned long long u64x8 __attribute__((ext_vector_type(8)));
    const u64x8 in = __builtin_bit_cast(u64x8, source);
    unsigned long long o0, o1, o2, o3, o4, o5, o6, o7;
    asm volatile("v_mov_b64 %0, %8\n\tv_mov_b64 %1, %9\n\tv_mov_b64 %2, %10\n\tv_mov_b64 %3, %11\n\t"
                 "v_mov_b64 %4, %12\n\tv_mov_b64 %5, %13\n\tv_mov_b64 %6, %14\n\tv_mov_b64 %7, %15"
                 : "=&v"(o0), "=&v"(o1), "=&v"(o2), "=&v"(o3), "=&v"(o4), "=&v"(o5), "=&v"(o6), "=&v"(o7)
                 : "v"(in[0]), "v"(in[1]), "v"(in[2]), "v"(in[3]), "v"(in[4]), "v"(in[5]), "v"(in[6]), "v"(in[7]));
    const u64x8 out = {o0, o1, o2, o3, o4, o5, o6, o7};
    target = __builtin_bit_cast(f32x16, out);
}

struct RowState {
    f32x16 o[DBLOCKS];
    float reference;  // point the exponentials are taken against, in log2 units (score * scale * log2 e)
    float row_sum;    // this lane's share of the normaliser
};

// Head room (log2 units) put between the first unit's maximum and the softmax
// reference of a walk, and the excess over the reference at which the reference
// is raised (2^80 per term leaves 2^47 of fp32 range for the sums).
constexpr float FAST_HEADROOM = 40.0f;
constexpr float FAST_LIMIT = 80.0f;

// Column of the output a lane's accumulator register stands for.
__device__ __forceinline__ constexpr int output_column(int d, int i4, int g) {
    return 32 * d + 8 * i4 + 4 * g;
}

// Normalised bf16 rows -> out_row(row) .. +512, staged through this wave's LDS
// region so that each store instruction writes one full 1 KB row.
template <typename RowPointer>
__device__ __forceinline__ void store_final(const RowState& state, float inverse, unsigned char* wave_lds, int lane,
                                            RowPointer out_row) {
    const int lq = lane % 32;
    const int g = lane / 32;
#pragma unroll
    for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
            u32x2 packed;
            packed.x = pack_bf16(state.o[d][4 * i4 + 0] * inverse, state.o[d][4 * i4 + 1] * inverse);
            packed.y = pack_bf16(state.o[d][4 * i4 + 2] * inverse, state.o[d][4 * i4 + 3] * inverse);
            *reinterpret_cast<u32x2*>(wave_lds + lq * EPILOGUE_PITCH + 2 * output_column(d, i4, g)) = packed;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
    __builtin_amdgcn_wave_barrier();
#pragma unroll 4
    for (int row = 0; row < 32; ++row) {
        bf16_t* destination = out_row(row);
        if (destination != nullptr) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(wave_lds + row * EPILOGUE_PITCH + 16 * lane);
            *reinterpret_cast<u32x4*>(destination + 8 * lane) = bits;
        }
    }
}

// A wave's unnormalised accumulators as bf16 in the registers' own order: 16-byte piece
// j of a lane holds registers 8*(j%2) .. 8*(j%2)+7 of column block j/2, and a wave
// instruction covers 1 KB of consecutive memory (32 KB per wave).  Nothing crosses
// lanes; the merge kernel reads the pieces back with the same lane numbering.
constexpr int PARTIAL_PIECES = 2 * DBLOCKS;
constexpr int PARTIAL_WAVE_BYTES = PARTIAL_PIECES * 64 * 16;

__device__ __forceinline__ void store_partial(const RowState& state, unsigned char* wave_block, int lane) {
#pragma unroll
    for (int j = 0; j < PARTIAL_PIECES; ++j) {
        const int d = j / 2;
        const int base = 8 * (j % 2);
        u32x4 packed;
#pragma unroll
        for (int k = 0; k < 4; ++k) packed[k] = pack_bf16(state.o[d][base + 2 * k], state.o[d][base + 2 * k + 1]);
        *reinterpret_cast<u32x4*>(wave_block + (j * 64 + lane) * 16) = packed;
    }
}

__device__ __forceinline__ void load_query(bf16x8 (&qf)[KSTEPS], const bf16_t* latent_row, const bf16_t* rope_row,
                                           bool valid, int g) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        u32x4 bits = {0, 0, 0, 0};
        if (valid) {
            const bf16_t* source = ks < RANK / 16 ? latent_row + 16 * ks + 8 * g : rope_row + 16 * (ks - RANK / 16) + 8 * g;
            bits = *reinterpret_cast<const u32x4*>(source);
        }
        qf[ks] = __builtin_bit_cast(bf16x8, bits);
    }
}

__device__ __forceinline__ void reset(RowState& state) {
#pragma unroll
    for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
        for (int i = 0; i < 16; ++i) state.o[d][i] = 0.f;
    }
    state.reference = -INFINITY;
    state.row_sum = 0.f;
}

// ----------------------------------------------------------------------------
// The walk: 32-key units, one matrix stream
// ----------------------------------------------------------------------------
//
// With one wave per SIMD nothing hides the vector arithmetic of the softmax unless the
// wave's own instruction stream does: a loop that computes scores, then probabilities,
// then the output update leaves the matrix pipeline idle through the middle third.  Here
// the key stream is consumed in units of 32 keys and the work of consecutive units is
// overlapped by hand:
//
//     step u:   S(u+1) = K(u+1) Q^T   36 MFMAs, with the softmax of S(u) -> P(u)
//                                     (exp2, sums, bf16 packing) issued between them
//               O^T  += V(u)^T P(u)   32 MFMAs, with the requests for unit u+3 between them
//
// one stream of 68 MFMAs per unit, each fed by one LDS fragment read through a small
// register ring that runs a few MFMAs ahead.  The scores of two units are live at a
// time (one being accumulated, one being turned into probabilities), so the steps
// alternate between two register sets.
//
// Units sit in a ring of four LDS slots (144 KB).
// Unit u+3 is requested during step u into the slot that unit u-1 left at the end of
// step u-1; unit u+1, requested two steps earlier, must have landed when step u
// starts: the wave waits for all but its youngest nine loads (its share of unit
// u+2) and the workgroup meets at one barrier per step.  Rows of a unit past the end
// of the sequence repeat the last valid row and their scores are masked, so nothing
// has to be cleared.

constexpr int UNIT = 32;
constexpr int UNIT_BYTES = UNIT * ROW_BYTES;              // 36 KB
constexpr int UNIT_SLOTS = 4;
constexpr int UNIT_LOADS = UNIT * CHUNKS / THREADS;       // 9 wave instructions of 1 KB per wave and unit
constexpr int STREAM_RING = 6;                            // fragments read ahead of the MFMA that takes them
static_assert(UNIT_LOADS * THREADS == UNIT * CHUNKS, "unit loads must divide evenly");

struct UnitSource {
    const bf16_t* base;      // first row of the unit (contiguous form; split form: of its latent part)
    const bf16_t* rope_base; // split form: first row of the unit's rope part
    unsigned lds_base;       // LDS byte offset of this wave's 9 KB of the unit's slot
    int key0;
    int row_limit;           // rows above it repeat it (>= 0: the unit holds a visible token)
    bool contiguous;         // the unit is one run of rows: no paging, or pages that hold whole units
    bool split;              // no paging, latent and rope parts in tensors of their own, offsets that fit 32 bits
    bool full;               // all 32 rows are visible tokens: the per-lane offsets are the same for every such unit
    bool enabled;
};

// Hands out the sources of consecutive units of one sequence.  The decode cache is packed
// (576-wide rows), so only paging decides the form.  When pages hold whole units, the ids of
// 64 consecutive pages of the sequence sit in one register (lane l: page first_page + l) and a
// unit finds its page with one lane read: a scalar load per unit would have its wait drain the
// LDS queue as well, in the middle of the fragment stream.
struct UnitCursor {
    int unit;                // the unit handed out next
    int page;                // its page (index into the sequence's block table) ...
    int within;              // ... and its place inside that page, in units
    int units_per_page;
    int first_page;          // page whose id lane 0 of `ids` holds
    int last_page;           // last page of the sequence with a visible token: no entry past it is read
    int ids;
    bool paged;
    bool contiguous;
    bool split;

    // Waits for the ids on the spot (the empty asm statement is their first use): a wait left to the
    // first lane read would sit on the path of every step and wait for the unit requests as well.
    __device__ __forceinline__ void load_ids(const KeyStream& keys, int from) {
        first_page = from;
        ids = keys.block_table[min(from + fresh_lane_id(), last_page)];
        asm volatile("" : "+v"(ids));
    }

    __device__ __forceinline__ void init(const KeyStream& keys, int first_unit, int last_token) {
        paged = keys.block_table != nullptr;
        contiguous = !paged || (keys.page_size % UNIT == 0);
        split = false;
        unit = __builtin_amdgcn_readfirstlane(first_unit);
        page = within = units_per_page = first_page = last_page = ids = 0;
        if (paged && contiguous) {
            units_per_page = __builtin_amdgcn_readfirstlane(keys.page_size / UNIT);
            page = __builtin_amdgcn_readfirstlane(first_unit / units_per_page);
            within = __builtin_amdgcn_readfirstlane(first_unit - page * units_per_page);
            last_page = __builtin_amdgcn_readfirstlane(last_token / keys.page_size);
            load_ids(keys, page);
        }
    }

    __device__ __forceinline__ UnitSource next(unsigned char* lds, const KeyStream& keys, int last_token, int wave,
                                               int unit_end) {
        UnitSource source;
        source.contiguous = contiguous;
        source.split = split;
        source.enabled = unit < unit_end;
        source.key0 = unit * UNIT;
        source.row_limit = last_token - source.key0;
        source.full = source.row_limit >= UNIT - 1;
        source.lds_base = __builtin_amdgcn_readfirstlane(lds_offset_of(lds) + ((unsigned)unit % UNIT_SLOTS) * UNIT_BYTES +
                                                         wave * (UNIT_LOADS * 1024));
        source.base = keys.latent;
        source.rope_base = keys.rope;
        if (split) {
            source.base = keys.latent + (size_t)source.key0 * keys.latent_stride;
            source.rope_base = keys.rope + (size_t)source.key0 * keys.rope_stride;
        }
        if (source.enabled && contiguous) {
            long long physical = source.key0;
            if (paged) {
                // enabled: the unit holds a visible token, so page <= last_page
                if (page - first_page >= 64) load_ids(keys, page);
                const int id = __builtin_amdgcn_readlane(ids, page - first_page);
                physical = (long long)id * keys.page_size + within * UNIT;
            }
            source.base = keys.latent + physical * WIDTH;
        }
        ++unit;
        if (paged && contiguous && ++within == units_per_page) {
            within = 0;
            ++page;
        }
        return source;
    }
};

// Per-lane offsets of the nine loads of a full unit (no row past the end of the sequence).
struct FullUnitOffsets {
    unsigned of[UNIT_LOADS];

    __device__ __forceinline__ void init(int wave, int lane) {
#pragma unroll
        for (int i = 0; i < UNIT_LOADS; ++i) {
            of[i] = index_math::contiguous_load_offset<ROW_BYTES, UNIT / 4>(wave, i, lane, UNIT - 1);
        }
    }
};

// Load number i (0..8) of a contiguous unit; i is a constant after unrolling.
__device__ __forceinline__ void issue_unit_load(const UnitSource& source, const FullUnitOffsets& offsets, int wave, int i,
                                                int lane) {
    const unsigned offset = source.full
        ? offsets.of[i]
        : index_math::contiguous_load_offset<ROW_BYTES, UNIT / 4>(wave, i, lane, source.row_limit);
    direct_load_16_offset_streaming(source.base, offset, source.lds_base + i * 1024);   // the cache is read once per call
}

// Load I of a unit whose latent and rope parts lie in tensors of their own, unpaged (`split`): a wave instruction
// covers at most two rows of the unit (compile-time boundary), and a lane's 16 bytes come from the one tensor or the
// other.  Row strides stay below 2^24 elements (the caller saw to that).
template <int I>
__device__ __forceinline__ void issue_split_load(const UnitSource& source, const KeyStream& keys, int wave, int lane) {
    constexpr int FIRST_ROW = (64 * I) / CHUNKS;                 // of the wave's eight rows: the row of lane 0
    constexpr int BOUNDARY = CHUNKS * (FIRST_ROW + 1) - 64 * I;   // first lane of the next row (64 or more: none)
    // what depends on the row is the same for all lanes of a row: two candidates, wave-uniform
    const int row = (UNIT / 4) * wave + FIRST_ROW;
    const int swizzle[2] = {swizzle_of_row(row), swizzle_of_row(row + 1)};
    const unsigned row_here[2] = {(unsigned)min(row, source.row_limit), (unsigned)min(row + 1, source.row_limit)};
    const bool second = BOUNDARY < 64 && lane >= BOUNDARY;
    const int position = lane + (64 * I - CHUNKS * FIRST_ROW) - (second ? CHUNKS : 0);
    const int chunk = position ^ (second ? swizzle[1] : swizzle[0]);
    const bool rope = chunk >= RANK / 8;
    // bytes from the first row of the unit's part in the lane's tensor (the bases of the source hold key0 * stride)
    const unsigned row_bytes = __umul24(second ? row_here[1] : row_here[0],
                                        rope ? 2u * (unsigned)keys.rope_stride : 2u * (unsigned)keys.latent_stride);
    const unsigned bytes = row_bytes + 16u * (unsigned)chunk - (rope ? 2u * RANK : 0u);
    const unsigned char* part = reinterpret_cast<const unsigned char*>(rope ? source.rope_base : source.base);
    direct_load_16(part + bytes, source.lds_base + I * 1024);
}

// All nine loads of a unit at once: the first units of a walk, and every unit of the
// general form (per-lane page lookup, or latent and rope parts in tensors of their own).
__device__ __forceinline__ void issue_unit(const UnitSource& source, const FullUnitOffsets& offsets, const KeyStream& keys,
                                           int wave) {
    if (!source.enabled) return;
    const int lane = fresh_lane_id();
    if (source.contiguous) {
#pragma unroll
        for (int i = 0; i < UNIT_LOADS; ++i) issue_unit_load(source, offsets, wave, i, lane);
        return;
    }
    if (source.split) {
        unrolled<0, UNIT_LOADS>([&](auto tag) { issue_split_load<decltype(tag)::value>(source, keys, wave, lane); });
        return;
    }
    const bool paged = keys.block_table != nullptr;
#pragma unroll 1
    for (int i = 0; i < UNIT_LOADS; ++i) {
        const int slot = 64 * i + lane;
        const int row = (UNIT / 4) * wave + slot / CHUNKS;
        const int chunk = (slot % CHUNKS) ^ swizzle_of_row(row);
        const int token = source.key0 + min(row, source.row_limit);
        long long physical = token;
        if (paged) {
            const int page = keys.block_table[token / keys.page_size];
            physical = (long long)page * keys.page_size + token % keys.page_size;
        }
        const bf16_t* address = chunk < RANK / 8 ? keys.latent + physical * keys.latent_stride + 8 * chunk
                                                 : keys.rope + physical * keys.rope_stride + 8 * (chunk - RANK / 8);
        direct_load_16(address, source.lds_base + i * 1024);
    }
}

// Per-lane byte offsets of the fragment reads inside a unit (rows 0..31 of 1152 bytes).
// K operand: row lane%32, 16-byte chunk 2*ks + g at position (2*ks + g) ^ f(row); the XOR
// only mixes the low three bits, so four offsets plus (ks/4)*128 reach every k-step.
// V^T operand through transposing reads: in a block of 16 lanes, lane s points at row
// 4*g + s/4 (+8 for the second read), columns 4*(s%4)..+3 of the 16-column group
// 16*(block%2); bit 2 of f moves a row's data by one 64-byte column block, which two
// offsets per read (even / odd column block) turn back into immediates.
struct UnitReads {
    unsigned k[4];
    unsigned v_first[2];
    unsigned v_second[2];

    __device__ __forceinline__ void init(int lane) {
        const int lq = lane % 32;
        const int g = lane / 32;
        const int swz = swizzle_of_row(lq);
#pragma unroll
        for (int j = 0; j < 4; ++j) k[j] = lq * ROW_BYTES + ((2 * j + g) ^ swz) * 16;
        const int s16 = lane % 16;
        const int block = lane / 16;
        const int row1 = 4 * g + s16 / 4;
        const int f1 = swizzle_of_row(row1);
        const int chunk_low = (2 * (block % 2) + (s16 % 4) / 2) ^ (f1 & 3);
        const int flip = 64 * ((row1 >> 1) & 1);
        const int lane1 = row1 * ROW_BYTES + chunk_low * 16 + 8 * (s16 & 1);
        const int lane2 = (row1 + 8) * ROW_BYTES + (chunk_low ^ 1) * 16 + 8 * (s16 & 1);
        v_first[0] = lane1 + flip;
        v_first[1] = lane1 - flip;
        v_second[0] = lane2 + flip;
        v_second[1] = lane2 - flip;
    }
};

typedef short unit_s16x4 __attribute__((ext_vector_type(4)));
typedef short unit_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) unit_s16x4* unit_tr_pointer;

template <int KS>
__device__ __forceinline__ bf16x8 unit_key_fragment(const unsigned char* unit, const UnitReads& reads) {
    return *reinterpret_cast<const bf16x8*>(unit + reads.k[KS % 4] + (KS / 4) * 128);
}

// 16-key step N (0, 1) of the unit, column block D (0..15)
template <int N, int D>
__device__ __forceinline__ bf16x8 unit_value_fragment(const unsigned char* unit, const UnitReads& reads) {
    constexpr int CONSTANT = N * 16 * ROW_BYTES + D * 64;
    const unit_s16x4 low = __builtin_amdgcn_ds_read_tr16_b64_v4i16((unit_tr_pointer)(unit + reads.v_first[D % 2] + CONSTANT));
    const unit_s16x4 high = __builtin_amdgcn_ds_read_tr16_b64_v4i16((unit_tr_pointer)(unit + reads.v_second[D % 2] + CONSTANT));
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(low, high, 0, 1, 2, 3, 4, 5, 6, 7));
}

// Scores of the unit at `unit` into `scores`, nothing overlapped (the first unit of a walk).
__device__ __forceinline__ void unit_scores(f32x16& scores, const bf16x8 (&qf)[KSTEPS], const unsigned char* unit,
                                            const UnitReads& reads) {
    bf16x8 ring[STREAM_RING];
    unrolled<0, STREAM_RING>([&](auto tag) { ring[decltype(tag)::value] = unit_key_fragment<decltype(tag)::value>(unit, reads); });
    unrolled<0, KSTEPS>([&](auto tag) {
        constexpr int I = decltype(tag)::value;
        if constexpr (I == 0) {
            score_mfma_first(scores, ring[0], qf[0]);
        } else if constexpr (I == KSTEPS - 1) {
            score_mfma_last(scores, ring[I % STREAM_RING], qf[I]);
        } else {
            score_mfma(scores, ring[I % STREAM_RING], qf[I]);
        }
        if constexpr (I + STREAM_RING < KSTEPS) ring[I % STREAM_RING] = unit_key_fragment<I + STREAM_RING>(unit, reads);
        __builtin_amdgcn_sched_barrier(0);
    });
}

__device__ __forceinline__ void mask_unit_scores(f32x16& scores, int key0, int tokens, int g) {
    if (key0 + UNIT > tokens) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int k = key0 + 8 * (i / 4) + 4 * g + (i % 4);
            if (k >= tokens) scores[i] = -INFINITY;
        }
    }
}

// A row's scores have outrun its reference by more than FAST_LIMIT: the reference of every such row of the
// wave moves to FAST_HEADROOM above the row's new maximum, and what the row has accumulated is scaled to
// match.  Next to never taken; when it is, some wave pays 256 multiplications per lane once.  The
// accumulators are scaled where they are (accumulation registers, read and written back by one asm
// statement each): any formulation that lets the compiler see a conditional assignment to them makes it
// copy all 256 at the join, on the path that never takes the branch as well.  The output MFMAs that wrote
// them were issued a whole unit ago; the wait states at the top cover the distance all the same.
__device__ __forceinline__ void raise_reference(RowState& state, float& offset, float unit_max) {
    const float raised = unit_max - offset > FAST_LIMIT ? unit_max + FAST_HEADROOM : offset;
    const float factor = __builtin_amdgcn_exp2f(offset - raised);   // 1 for the rows that stay
    offset = raised;
    state.reference = raised;
    state.row_sum *= factor;
    asm volatile("s_nop 15\n\ts_nop 3");
#pragma unroll
    for (int d = 0; d < DBLOCKS; ++d) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float value = state.o[d][i];
            float moved;
            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                         : "+a"(value), "=&v"(moved)
                         : "v"(factor));
            state.o[d][i] = value;
        }
    }
}

// One step of the stream: the probabilities of the unit at `current` (its scores are in
// `scores`), the scores of the unit at `next` into `next_scores` if HAS_NEXT, the output
// update with `current`, and the requests for `request`.
template <bool HAS_NEXT>
__device__ __forceinline__ void unit_step(RowState& state, f32x16& scores, f32x16& next_scores,
                                          const bf16x8 (&qf)[KSTEPS], const UnitReads& reads,
                                          const unsigned char* current, const unsigned char* next, int key0, int tokens,  // tokens: of the lane's row
                                          float c, const UnitSource& request, const FullUnitOffsets& offsets,
                                          const KeyStream& keys, int wave) {
    constexpr int SCORE_MFMAS = HAS_NEXT ? KSTEPS : 0;
    constexpr int COUNT = SCORE_MFMAS + 2 * DBLOCKS;
    const int lane = fresh_lane_id();

    // fragment I of the stream: the K fragments of the next unit, then the V fragments of this one
    auto fragment = [&](auto tag) -> bf16x8 {
        constexpr int I = decltype(tag)::value;
        if constexpr (I < SCORE_MFMAS) {
            return unit_key_fragment<I>(next, reads);
        } else {
            return unit_value_fragment<(I - SCORE_MFMAS) / DBLOCKS, (I - SCORE_MFMAS) % DBLOCKS>(current, reads);
        }
    };
    bf16x8 ring[STREAM_RING];
    unrolled<0, STREAM_RING>([&](auto tag) { ring[decltype(tag)::value] = fragment(tag); });

    mask_unit_scores(scores, key0, tokens, lane / 32);

    float unit_max;
    u32x4 probabilities[2];
    float offset = state.reference;
    // The softmax in 33 pieces of one to three instructions, spread over the score MFMAs.  Plain
    // arithmetic has no place of its own in the instruction order (the compiler would gather all of
    // it next to its last use, behind the score MFMAs); passing a piece's inputs and results through
    // empty volatile asm statements ties it to the spot between the two hand-issued MFMAs around it.
    auto here = [](float& value) { asm volatile("" : "+v"(value)); };
    float exponentials[16];
    auto softmax_piece = [&](auto tag) {
        constexpr int I = decltype(tag)::value;
        if constexpr (I < 8) {
            float first = scores[2 * I];
            here(first);
            unit_max = I == 0 ? fmaxf(first, scores[1]) : fmaxf(unit_max, fmaxf(first, scores[2 * I + 1]));
            here(unit_max);
        } else if constexpr (I == 8) {
            unit_max = half_wave_max(unit_max) * c;
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(unit_max - offset > FAST_LIMIT) != 0, 0)) {
                raise_reference(state, offset, unit_max);
            }
        } else if constexpr (I < 25) {
            constexpr int E = I - 9;
            float score = scores[E];
            here(score);
            const float p = __builtin_amdgcn_exp2f(fmaf(score, c, -offset));
            state.row_sum += p;
            // The sum is what gets tied down, never the exponential itself: an asm statement that
            // takes the result of v_exp hides from the compiler that its next reader follows a
            // transcendental, and the wait state that pairing needs would go missing.
            here(state.row_sum);
            exponentials[E] = p;
        } else if constexpr (I < 33) {
            constexpr int K = I - 25;
            float low = exponentials[2 * K];
            here(low);
            float packed = __uint_as_float(pack_bf16(low, exponentials[2 * K + 1]));
            here(packed);
            probabilities[K / 4][K % 4] = __float_as_uint(packed);
        }
    };
    if constexpr (!HAS_NEXT) {
        unrolled<0, 33>(softmax_piece);   // the last unit: no score products to hide it behind
    }
    if (request.enabled && !request.contiguous && !request.split) issue_unit(request, offsets, keys, wave);

    unrolled<0, COUNT>([&](auto tag) {
        constexpr int I = decltype(tag)::value;
        if constexpr (I < SCORE_MFMAS) {
            if constexpr (I == 0) {
                score_mfma_first(next_scores, ring[0], qf[0]);
            } else if constexpr (I == KSTEPS - 1) {
                score_mfma_last(next_scores, ring[I % STREAM_RING], qf[I]);   // its wait states pass while it executes
            } else {
                score_mfma(next_scores, ring[I % STREAM_RING], qf[I]);
            }
        } else {
            constexpr int J = I - SCORE_MFMAS;
            state.o[J % DBLOCKS] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                ring[I % STREAM_RING], __builtin_bit_cast(bf16x8, probabilities[J / DBLOCKS]), state.o[J % DBLOCKS], 0, 0, 0);
        }
        if constexpr (I + STREAM_RING < COUNT) ring[I % STREAM_RING] = fragment(std::integral_constant<int, I + STREAM_RING>{});
        if constexpr (HAS_NEXT && I < 33) softmax_piece(tag);
        // the requests go between the output MFMAs, which leave more issue slots free than the score MFMAs
        if constexpr (HAS_NEXT && I >= SCORE_MFMAS && (I - SCORE_MFMAS) % 3 == 1 && (I - SCORE_MFMAS) / 3 < UNIT_LOADS) {
            if (request.enabled && request.contiguous) issue_unit_load(request, offsets, wave, (I - SCORE_MFMAS) / 3, lane);
            if (request.enabled && request.split) issue_split_load<(I - SCORE_MFMAS) / 3>(request, keys, wave, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
    });
}

// Walk tiles [tile_begin, tile_end) of one sequence of keys for the 128 rows of this workgroup
// with the unit stream, from cleared accumulators (see raise_reference for what happens when a
// row outruns its softmax reference).  Decode: the rows are the heads of one sequence, each sees
// all `tokens` keys of the packed cache.  PREFILL: the rows are (token, head) pairs, a lane's row
// sees the first `row_tokens` <= `tokens` keys (at least one), and the latent and rope parts of
// the keys lie in tensors of their own.
template <bool PREFILL>
__device__ __forceinline__ void walk_units(RowState& state, const bf16_t* query_latent_row, const bf16_t* query_rope_row,
                                           bool valid, unsigned char* lds, const KeyStream& keys, int tile_begin,
                                           int tile_end, int tokens, int row_tokens, float c, int tid, bool cold) {
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int last_token = tokens - 1;
    const int unit_begin = (BN / UNIT) * tile_begin;
    const int unit_end = min((BN / UNIT) * tile_end, (tokens + UNIT - 1) / UNIT);   // > unit_begin

    // The first three units and the query rows.  In the middle of a kernel one round trip brings them all.  At the
    // start of the kernel (`cold`) every workgroup asks at once and the answers come at the rate of the memory, not
    // of its latency: then only what the first scores need is asked for first, the rest once that has arrived.
    // The query rows are asked for before the page ids of the cursor, whose wait then covers both round trips
    // (the ids are needed before the first unit can be requested; the rows before its scores).
    bf16x8 qf[KSTEPS];
    load_query(qf, query_latent_row, query_rope_row, valid, (tid % 64) / 32);
    UnitCursor cursor;
    cursor.init(keys, unit_begin, last_token);
    if constexpr (PREFILL) {
        cursor.contiguous = false;   // latent and rope parts come from tensors of their own
        // 32 rows of a unit times the row stride, in bytes, as a 32-bit lane offset
        cursor.split = keys.block_table == nullptr && keys.latent_stride < ((size_t)1 << 24) &&
                       keys.rope_stride < ((size_t)1 << 24);
    }
    const int visible = PREFILL ? row_tokens : tokens;   // keys the lane's row sees
    FullUnitOffsets offsets;
    offsets.init(wave, fresh_lane_id());
    issue_unit(cursor.next(lds, keys, last_token, wave, unit_end), offsets, keys, wave);
    const UnitSource second = cursor.next(lds, keys, last_token, wave, unit_end);
    const UnitSource third = cursor.next(lds, keys, last_token, wave, unit_end);
    if (!cold) issue_unit(second, offsets, keys, wave);
    if (!cold) issue_unit(third, offsets, keys, wave);
    reset(state);
    UnitReads reads;
    reads.init(fresh_lane_id());
    auto slot_of = [&](int unit) { return lds + ((unsigned)unit % UNIT_SLOTS) * UNIT_BYTES; };

    wait_vector_memory<0>();
    workgroup_barrier();
    if (cold) {
        issue_unit(second, offsets, keys, wave);
        issue_unit(third, offsets, keys, wave);
    }
    // scores of the first unit, and the reference every exponential of this walk is taken against
    f32x16 scores_a, scores_b;
    unit_scores(scores_a, qf, slot_of(unit_begin), reads);
    {
        mask_unit_scores(scores_a, unit_begin * UNIT, visible, fresh_lane_id() / 32);
        float first_max = scores_a[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) first_max = fmaxf(first_max, scores_a[i]);
        state.reference = half_wave_max(first_max) * c + FAST_HEADROOM;
    }

    auto synchronise = [&](int at) {
        // unit at + 1 (requested during step at - 2, or before the loop) has landed; only this wave's share of
        // unit at + 2, requested later, may still be in flight
        if (at + 2 < unit_end) {
            wait_vector_memory<UNIT_LOADS>();
        } else {
            wait_vector_memory<0>();
        }
        workgroup_barrier();   // ... and everybody's share; every wave has left step at - 1
    };
    int unit = unit_begin;
    for (; unit + 1 < unit_end; ++unit) {
        synchronise(unit);
        unit_step<true>(state, scores_a, scores_b, qf, reads, slot_of(unit), slot_of(unit + 1), unit * UNIT, visible, c,
                        cursor.next(lds, keys, last_token, wave, unit_end), offsets, keys, wave);
        // the next unit's scores take the place of this unit's (eight moves against a stream of 68 MFMAs)
        move_scores(scores_a, scores_b);
    }
    UnitSource nothing = {};
    unit_step<false>(state, scores_a, scores_b, qf, reads, slot_of(unit), slot_of(unit), unit * UNIT, visible, c, nothing,
                     offsets, keys, wave);
    workgroup_barrier();   // the slots are free: the caller stages its results through them
}

__device__ __forceinline__ int tiles_of(int length) {
    return (max(length, 0) + BN - 1) / BN;
}

// ----------------------------------------------------------------------------
// decode
// ----------------------------------------------------------------------------

using index_math::PLAN_HEADER;
using index_math::PLAN_OVERHEAD;
using index_math::PLAN_RANGES;
using index_math::PLAN_TOTAL;
using index_math::PLAN_WHOLE;
using index_math::PLAN_WORKGROUPS;

// One workgroup turns the lengths into the plan (index_math.h): the prefix of positions
// (tiles plus the per-sequence overhead when sequences are cut), the first sequence of
// each of the `workgroups` ranges.  Any batch size: the scan carries over chunks of
// THREADS lengths.
__global__ __launch_bounds__(THREADS) void mla_decode_plan_kernel(int* __restrict__ plan,
                                                                  const int* __restrict__ cache_lengths, int batch_size,
                                                                  int workgroups, int whole_sequences) {
    __shared__ int wave_totals[THREADS / 64];
    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = tid / 64;
    int* prefix = plan + index_math::plan_prefix_at();
    int* first_sequence = plan + index_math::plan_first_sequence_at(batch_size);

    const int overhead = whole_sequences ? 0 : index_math::SEGMENT_OVERHEAD;
    int carry = 0;
    if (tid == 0) prefix[0] = 0;
    for (int base = 0; base < batch_size; base += THREADS) {
        const int index = base + tid;
        int value = index < batch_size ? index_math::positions_of(tiles_of(cache_lengths[index]), overhead) : 0;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const int other = __shfl_up(value, offset);
            if (lane >= offset) value += other;
        }
        if (lane == 63) wave_totals[wave] = value;
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < THREADS / 64; ++w) {
            const int t = wave_totals[w];
            if (w < wave) before += t;
            total += t;
        }
        if (index < batch_size) prefix[index + 1] = carry + before + value;
        carry += total;
        __syncthreads();
    }
    const int total = carry;
    const int ranges = index_math::ranges_of(total, workgroups);
    if (tid == 0) {
        plan[PLAN_TOTAL] = total;
        plan[PLAN_WORKGROUPS] = workgroups;
        plan[PLAN_OVERHEAD] = overhead;
        plan[PLAN_RANGES] = ranges;
        plan[PLAN_WHOLE] = whole_sequences;
    }
    __syncthreads();   // the prefix written above is read back below
    for (int w = tid; w < workgroups; w += THREADS) {
        int sequence = w;
        if (!whole_sequences) {
            if (w >= ranges) {
                first_sequence[w] = batch_size;
                continue;
            }
            const int begin = index_math::range_begin_of(total, ranges, w);
            // first sequence whose positions reach past `begin`
            int low = 0, high = batch_size;
            while (low < high) {
                const int mid = (low + high) / 2;
                if (prefix[mid + 1] <= begin) low = mid + 1; else high = mid;
            }
            sequence = low;
        }
        first_sequence[w] = sequence;
    }
}

constexpr int SELF_PLAN_BATCH = THREADS;   // sequences a workgroup turns into a plan by itself

// The decode kernel: every workgroup walks its range of the work list (see index_math.h).
//
// Workspace: slot workgroup + sequence holds, for a segment that is only part of its
// sequence, the bf16 accumulators of every wave (store_partial order, 32 KB per wave,
// waves numbered over all head groups) followed by (reference, sum) per head.
__global__ __launch_bounds__(THREADS) void mla_decode_split_kernel(
    bf16_t* __restrict__ output, float* __restrict__ logsumexp, const bf16_t* __restrict__ query,
    const bf16_t* __restrict__ paged_kv_cache, const int* __restrict__ block_table,
    const int* __restrict__ cache_lengths, float* __restrict__ workspace, int* __restrict__ plan, int batch_size,
    int heads, int page_size, int pages_per_sequence, long long slot_floats, int padded_rows, float scale,
    int own_workgroups, int own_whole) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ int own_prefix[SELF_PLAN_BATCH + 1];
    __shared__ int own_lengths[SELF_PLAN_BATCH];   // saves the walk a round trip to memory for its sequence's length
    __shared__ int own_wave_totals[THREADS / 64];

    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = tid / 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    // Workgroups go to the eight XCDs round-robin by linear id.  Neighbouring ranges are mostly parts of the same
    // sequence and fetch the same query rows, so each XCD takes a run of consecutive ranges and its L2 serves all but
    // the first of those fetches.
    const int workgroup = gridDim.x % 8 == 0 ? (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8) : (int)blockIdx.x;
    const int head_group = blockIdx.y;
    const int head0 = head_group * ROWS;
    const float c = uniform(scale * LOG2E);

    // The plan: read from memory (own_workgroups == 0: the caller's, or one mla_decode_plan_kernel has just built),
    // or, for a batch that one workgroup scans in one go, worked out here by every workgroup for itself, which
    // saves the call a kernel launch.  The first workgroup then also leaves what the merge kernel reads of it.
    int total, overhead, ranges;
    bool whole_sequences;
    const int* prefix;
    if (own_workgroups > 0) {
        whole_sequences = own_whole != 0;
        overhead = whole_sequences ? 0 : index_math::SEGMENT_OVERHEAD;
        const int own_length = tid < batch_size ? cache_lengths[tid] : 0;
        own_lengths[tid] = own_length;
        int value = tid < batch_size ? index_math::positions_of(tiles_of(own_length), overhead) : 0;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const int other = __shfl_up(value, offset);
            if (lane >= offset) value += other;
        }
        if (lane == 63) own_wave_totals[wave] = value;
        if (tid == 0) own_prefix[0] = 0;
        __syncthreads();
        int before = 0;
#pragma unroll
        for (int w = 0; w < THREADS / 64; ++w) {
            if (w < wave) before += own_wave_totals[w];
        }
        if (tid < batch_size) own_prefix[tid + 1] = before + value;
        __syncthreads();
        // what comes out of LDS is the same in every lane, which the compiler cannot know: say so, or everything
        // computed from it (the base addresses of the unit requests among it) ends up in vector registers
        total = __builtin_amdgcn_readfirstlane(own_prefix[batch_size]);
        ranges = index_math::ranges_of(total, own_workgroups);
        prefix = own_prefix;
        if (blockIdx.x == 0 && blockIdx.y == 0) {
            if (tid == 0) {
                plan[PLAN_TOTAL] = total;
                plan[PLAN_WORKGROUPS] = own_workgroups;
                plan[PLAN_OVERHEAD] = overhead;
                plan[PLAN_WHOLE] = own_whole;
                plan[PLAN_RANGES] = ranges;
            }
            if (tid <= batch_size) plan[index_math::plan_prefix_at() + tid] = own_prefix[tid];
        }
    } else {
        total = plan[PLAN_TOTAL];
        overhead = plan[PLAN_OVERHEAD];
        whole_sequences = plan[PLAN_WHOLE] != 0;
        ranges = plan[PLAN_RANGES];
        prefix = plan + index_math::plan_prefix_at();
    }

    int range_begin, range_end;
    if (whole_sequences) {
        range_begin = __builtin_amdgcn_readfirstlane(prefix[workgroup]);
        range_end = __builtin_amdgcn_readfirstlane(prefix[workgroup + 1]);
    } else {
        if (workgroup >= ranges) return;
        range_begin = index_math::range_begin_of(total, ranges, workgroup);
        range_end = index_math::range_begin_of(total, ranges, workgroup + 1);
    }
    if (range_begin >= range_end) return;
    int sequence;
    if (own_workgroups > 0 && !whole_sequences) {
        // first sequence whose positions reach past range_begin
        int low = 0, high = batch_size;
        while (low < high) {
            const int mid = (low + high) / 2;
            if (__builtin_amdgcn_readfirstlane(prefix[mid + 1]) <= range_begin) low = mid + 1; else high = mid;
        }
        sequence = low;
    } else if (own_workgroups > 0) {
        sequence = workgroup;
    } else {
        sequence = plan[index_math::plan_first_sequence_at(batch_size) + workgroup];
    }

    const int head = head0 + 32 * wave + lq;
    const bool valid = head < heads;
    const bool wave_active = head0 + 32 * wave < heads;
    const int row = valid ? head : 0;
    unsigned char* wave_lds = lds + wave * 32 * EPILOGUE_PITCH;
    const size_t partial_wave_offset = (size_t)(head_group * (ROWS / 32) + wave) * PARTIAL_WAVE_BYTES;
    const size_t stats_offset = (size_t)padded_rows * (RANK / 2);   // in floats, behind the bf16 rows of a slot

    RowState state;
    int position = range_begin;
    while (position < range_end) {
        const int sequence_begin = __builtin_amdgcn_readfirstlane(prefix[sequence]);
        const int sequence_end = __builtin_amdgcn_readfirstlane(prefix[sequence + 1]);
        const int segment_end = min(range_end, sequence_end);
        if (segment_end <= position) {  // a sequence without tiles (length < 1) owns nothing
            ++sequence;
            continue;
        }
        int tile_begin, tile_end;
        index_math::tiles_in_positions(position, segment_end, sequence_begin, overhead, tile_begin, tile_end);
        // no tiles: the range ends among the positions that stand for the sequence's overhead
        if (tile_end <= tile_begin) {
            position = segment_end;
            ++sequence;
            continue;
        }
        const int tokens = own_workgroups > 0 ? __builtin_amdgcn_readfirstlane(own_lengths[sequence]) : cache_lengths[sequence];
        const bool whole = tile_begin == 0 && tile_end == sequence_end - sequence_begin - overhead;
        const bf16_t* query_row = query + ((size_t)sequence * heads + row) * WIDTH;

        KeyStream keys;
        keys.latent = paged_kv_cache;
        keys.rope = paged_kv_cache + RANK;
        keys.latent_stride = WIDTH;
        keys.rope_stride = WIDTH;
        keys.block_table = block_table + (size_t)sequence * pages_per_sequence;
        keys.page_size = page_size;
        walk_units<false>(state, query_row, query_row + RANK, valid, lds, keys, tile_begin, tile_end, tokens, tokens, c, tid,
                          position == range_begin);
        const float total_sum = half_wave_sum(state.row_sum);

        if (whole) {
            if (wave_active) {
                if (valid && g == 0) {
                    logsumexp[(size_t)sequence * heads + head] = (state.reference + __builtin_amdgcn_logf(total_sum)) * LN2;
                }
                store_final(state, 1.0f / total_sum, wave_lds, lane, [&](int r) -> bf16_t* {
                    const int h = head0 + 32 * wave + r;
                    return h < heads ? output + ((size_t)sequence * heads + h) * RANK : nullptr;
                });
            }
        } else if (wave_active) {
            float* slot = workspace + ((size_t)workgroup + sequence) * slot_floats;
            if (valid && g == 0) {
                slot[stats_offset + 2 * head] = state.reference;
                slot[stats_offset + 2 * head + 1] = total_sum;
            }
            store_partial(state, reinterpret_cast<unsigned char*>(slot) + partial_wave_offset, lane);
        }
        __syncthreads();  // the staging region is about to be overwritten by the next segment's tiles
        position = segment_end;
        ++sequence;
    }
}

// Merge the parts of every sequence that was cut by a range boundary.  One wave per
// (sequence, wave of 32 heads, quarter of the 512 columns): it reads its share of every
// part in the order the registers of the split kernel held it (same lane numbering),
// so lane l ends up with head l % 32 and, per column block d, the columns
// output_column(d, i4, l / 32) + 0..3; the results go through LDS to leave as 16-byte
// pieces of output rows.
constexpr int MERGE_QUARTERS = 4;
constexpr int MERGE_PIECES = PARTIAL_PIECES / MERGE_QUARTERS;       // 8 pieces of 16 bytes per lane and part
constexpr int MERGE_COLUMNS = RANK / MERGE_QUARTERS;                // 128
constexpr int MERGE_PITCH = MERGE_COLUMNS * 2 + 16;                  // bytes per staged row

__global__ __launch_bounds__(64) void mla_decode_merge_kernel(bf16_t* __restrict__ output, float* __restrict__ logsumexp,
                                                              const float* __restrict__ workspace, int* __restrict__ plan,
                                                              int batch_size, int heads, long long slot_floats,
                                                              int padded_rows) {
    __shared__ __attribute__((aligned(16))) unsigned char staging[32 * MERGE_PITCH];
    const int lane = threadIdx.x;
    const int lq = lane % 32;
    const int g = lane / 32;
    const int quarter = blockIdx.x % MERGE_QUARTERS;
    const int wave_block = blockIdx.x / MERGE_QUARTERS;   // 32 heads, numbered over all head groups
    const int sequence = blockIdx.y;

    const int total = plan[PLAN_TOTAL];
    const int workgroups = plan[PLAN_WORKGROUPS];
    const int overhead = plan[PLAN_OVERHEAD];
    const int* prefix = plan + index_math::plan_prefix_at();
    const int sequence_begin = prefix[sequence];
    const int sequence_end = prefix[sequence + 1];
    if (sequence_end <= sequence_begin) return;   // no tiles: nothing was computed for it
    int first, last;
    index_math::ranges_of_sequence(total, plan[PLAN_RANGES], sequence_begin, sequence_end - sequence_begin, overhead, first, last);
    if (first == last) return;                    // finished in place by the split kernel

    const int head = 32 * wave_block + lq;
    const bool valid = head < heads;
    const size_t stats_offset = (size_t)padded_rows * (RANK / 2);
    const size_t pieces_offset = (size_t)wave_block * PARTIAL_WAVE_BYTES + (size_t)(quarter * MERGE_PIECES * 64 + lane) * 16;

    float reference = -INFINITY;
    for (int w = first; w <= last; ++w) {
        const float* part = workspace + ((size_t)w + sequence) * slot_floats;
        if (valid) reference = fmaxf(reference, part[stats_offset + 2 * head]);
    }
    float normaliser = 0.f;
    float sums[MERGE_PIECES][8];
#pragma unroll
    for (int j = 0; j < MERGE_PIECES; ++j) {
#pragma unroll
        for (int k = 0; k < 8; ++k) sums[j][k] = 0.f;
    }
    for (int w = first; w <= last; ++w) {
        const float* part = workspace + ((size_t)w + sequence) * slot_floats;
        float weight = 0.f;
        if (valid) {
            weight = __builtin_amdgcn_exp2f(part[stats_offset + 2 * head] - reference);
            normaliser = fmaf(weight, part[stats_offset + 2 * head + 1], normaliser);
        }
        const unsigned char* pieces = reinterpret_cast<const unsigned char*>(part) + pieces_offset;
#pragma unroll
        for (int j = 0; j < MERGE_PIECES; ++j) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(pieces + j * 1024);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                sums[j][2 * k] = fmaf(weight, __uint_as_float(bits[k] << 16), sums[j][2 * k]);
                sums[j][2 * k + 1] = fmaf(weight, __uint_as_float(bits[k] & 0xffff0000u), sums[j][2 * k + 1]);
            }
        }
    }
    const float inverse = valid ? 1.0f / normaliser : 0.f;
    // piece j of the quarter is registers 8*(j%2) .. +7 of column block d = 4*quarter + j/2: two runs of
    // four columns, output_column(d, 2*(j%2), g) and output_column(d, 2*(j%2) + 1, g)
#pragma unroll
    for (int j = 0; j < MERGE_PIECES; ++j) {
#pragma unroll
        for (int run = 0; run < 2; ++run) {
            u32x2 packed;
            packed.x = pack_bf16(sums[j][4 * run] * inverse, sums[j][4 * run + 1] * inverse);
            packed.y = pack_bf16(sums[j][4 * run + 2] * inverse, sums[j][4 * run + 3] * inverse);
            const int column = output_column(j / 2, 2 * (j % 2) + run, g);   // within the quarter's 128 columns
            *reinterpret_cast<u32x2*>(staging + lq * MERGE_PITCH + 2 * column) = packed;
        }
    }
    __syncthreads();
    // 32 rows x 256 bytes: 16 lanes per row, four rows per pass
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
        const int r = 4 * pass + lane / 16;
        const int h = 32 * wave_block + r;
        if (h < heads) {
            const u32x4 bits = *reinterpret_cast<const u32x4*>(staging + r * MERGE_PITCH + 16 * (lane % 16));
            *reinterpret_cast<u32x4*>(output + ((size_t)sequence * heads + h) * RANK + quarter * MERGE_COLUMNS + 8 * (lane % 16)) = bits;
        }
    }
    if (quarter == 0 && valid && g == 0) {
        logsumexp[(size_t)sequence * heads + head] = (reference + __builtin_amdgcn_logf(normaliser)) * LN2;
    }
}

// ----------------------------------------------------------------------------
// absorbed causal prefill forward
// ----------------------------------------------------------------------------

__global__ __launch_bounds__(THREADS) void mla_absorbed_forward_kernel(
    bf16_t* __restrict__ output, float* __restrict__ logsumexp, const bf16_t* __restrict__ query_latent,
    const bf16_t* __restrict__ query_rope, const bf16_t* __restrict__ kv_latent, const bf16_t* __restrict__ key_rope,
    int sequence_length, int heads, int row_blocks, float scale) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid % 64;
    const int wave = tid / 64;
    const int lq = lane % 32;
    const int g = lane / 32;
    const float c = uniform(scale * LOG2E);

    // heaviest (latest) row blocks first
    const int batch = blockIdx.x / row_blocks;
    const int row_block = row_blocks - 1 - blockIdx.x % row_blocks;
    const long long rows = (long long)sequence_length * heads;   // (token, head) pairs of one batch element
    const long long row0 = (long long)row_block * ROWS;
    const long long row = row0 + 32 * wave + lq;
    const bool valid = row < rows;
    const bool wave_active = row0 + 32 * wave < rows;
    const int token = valid ? (int)(row / heads) : 0;
    const int head = valid ? (int)(row % heads) : 0;
    const long long global_row = (long long)batch * rows + (valid ? row : 0);

    RowState state;

    const long long last_row = min(rows, row0 + ROWS) - 1;
    const int visible = (int)(last_row / heads) + 1;  // keys any row of this block may see
    KeyStream keys;
    keys.latent = kv_latent + (size_t)batch * sequence_length * RANK;
    keys.rope = key_rope + (size_t)batch * sequence_length * ROPE;
    keys.latent_stride = RANK;
    keys.rope_stride = ROPE;
    keys.block_table = nullptr;
    keys.page_size = 0;
    walk_units<true>(state, query_latent + global_row * RANK, query_rope + global_row * ROPE, valid, lds, keys, 0,
                     tiles_of(visible), visible, valid ? token + 1 : visible, c, tid, true);

    if (!wave_active) return;
    const float total_sum = half_wave_sum(state.row_sum);
    if (valid && g == 0) {
        logsumexp[((size_t)batch * heads + head) * sequence_length + token] =
            (state.reference + __builtin_amdgcn_logf(total_sum)) * LN2;
    }
    unsigned char* wave_lds = lds + wave * 32 * EPILOGUE_PITCH;
    store_final(state, 1.0f / total_sum, wave_lds, lane, [&](int r) -> bf16_t* {
        const long long rr = row0 + 32 * wave + r;
        return rr < rows ? output + ((long long)batch * rows + rr) * RANK : nullptr;
    });
}

constexpr int LDS_BYTES = UNIT_SLOTS * UNIT_BYTES;

template <typename Kernel>
void allow_large_lds(Kernel kernel) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  LDS_BYTES));
}

// The count decides how many ranges a call's work list is cut into, so it is clamped to the bound
// the plan size below is computed for.
int compute_units() {
    return std::min(std::max(hip_common::compute_units_of_current_device(), 1), index_math::PLAN_MAX_WORKGROUPS);
}

}  // namespace

std::size_t mla_decode_plan_elements(int batch_size, int /*heads*/, int /*splits*/) {
    // Pure arithmetic, no device needed (as the reference's workspace size, kernels/attention/mla/sm89.cu:539-541):
    // room for the plan of any device this library runs on.
    return static_cast<std::size_t>(index_math::plan_elements_bound(batch_size));
}

void mla_decode_plan_dispatch(int* plan, const int* cache_lengths, int batch_size, int heads, int splits,
                              hipStream_t stream) {
    const index_math::DecodeLayout layout = index_math::decode_layout(batch_size, heads, splits, compute_units(), ROWS, RANK);
    hipLaunchKernelGGL(mla_decode_plan_kernel, dim3(1), dim3(THREADS), 0, stream, plan, cache_lengths, batch_size,
                       layout.workgroups, layout.whole_sequences);
    HIP_CHECK(hipGetLastError());
}

void mla_decode_dispatch(bf16_t* output, float* logsumexp, const bf16_t* query, const bf16_t* paged_kv_cache,
                         const int* block_table, const int* cache_lengths, float* workspace, int* plan,
                         int batch_size, int heads, int page_size, int pages_per_sequence, int splits, float scale,
                         hipStream_t stream) {
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) {
        throw std::invalid_argument("MLA decode requires a workspace aligned to 16 bytes");
    }
    static hip_common::OncePerDevice prepared;
    prepared.run([] { allow_large_lds(mla_decode_split_kernel); });
    // How the caller's B*H*splits*(C+2) floats are used: index_math::decode_layout.
    const index_math::DecodeLayout layout = index_math::decode_layout(batch_size, heads, splits, compute_units(), ROWS, RANK);
    int own_workgroups = 0;
    if (plan == nullptr) {
        // no plan from the caller: this call's own, behind the partial-result slots -- built by the decode kernel
        // itself when one workgroup can scan the batch, by the plan kernel otherwise
        plan = reinterpret_cast<int*>(workspace + layout.plan_offset);
        if (batch_size <= SELF_PLAN_BATCH) {
            own_workgroups = layout.workgroups;
        } else {
            hipLaunchKernelGGL(mla_decode_plan_kernel, dim3(1), dim3(THREADS), 0, stream, plan, cache_lengths, batch_size,
                               layout.workgroups, layout.whole_sequences);
            HIP_CHECK(hipGetLastError());
        }
    }
    const int padded_rows = (heads + 31) / 32 * 32;
    const dim3 grid(layout.workgroups, layout.head_groups);
    hipLaunchKernelGGL(mla_decode_split_kernel, grid, dim3(THREADS), LDS_BYTES, stream, output, logsumexp, query,
                       paged_kv_cache, block_table, cache_lengths, workspace, plan, batch_size, heads, page_size,
                       pages_per_sequence, layout.slot_floats, padded_rows, scale, own_workgroups, layout.whole_sequences);
    HIP_CHECK(hipGetLastError());
    if (!layout.whole_sequences) {
        hipLaunchKernelGGL(mla_decode_merge_kernel, dim3(MERGE_QUARTERS * (padded_rows / 32), batch_size), dim3(64), 0,
                           stream, output, logsumexp, workspace, plan, batch_size, heads, layout.slot_floats,
                           padded_rows);
        HIP_CHECK(hipGetLastError());
    }
}

void mla_absorbed_forward_dispatch(bf16_t* output, float* logsumexp, const bf16_t* query_latent,
                                   const bf16_t* query_rope, const bf16_t* kv_latent, const bf16_t* key_rope,
                                   int batch_size, int sequence_length, int heads, float scale, hipStream_t stream) {
    static hip_common::OncePerDevice prepared;
    prepared.run([] { allow_large_lds(mla_absorbed_forward_kernel); });
    const long long rows = (long long)sequence_length * heads;
    const long long row_blocks = (rows + ROWS - 1) / ROWS;
    if (row_blocks * batch_size > 0x7fffffffLL) {
        throw std::invalid_argument("MLA forward: batch*tokens*heads exceeds the grid limit");
    }
    hipLaunchKernelGGL(mla_absorbed_forward_kernel, dim3((unsigned)(row_blocks * batch_size)), dim3(THREADS), LDS_BYTES,
                       stream, output, logsumexp, query_latent, query_rope, kv_latent, key_rope, sequence_length, heads,
                       (int)row_blocks, scale);
    HIP_CHECK(hipGetLastError());
}

}  // namespace dscuda
