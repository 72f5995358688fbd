// Integer arithmetic of the attention kernels that decides where data lives and
// which workgroup does what: LDS chunk permutations, tile-request offsets, the
// position of a dS block in the backward workspace, the work order of the
// persistent forward kernel and the split of the decode tile list.  Kept free
// of anything device-specific so that the same definitions compile for the
// host, where tests enumerate them exhaustively (coverage, uniqueness,
// fast path == general path).
#pragma once

#if defined(__HIPCC__)
#define DSCUDA_HOST_DEVICE __host__ __device__
#else
#define DSCUDA_HOST_DEVICE
#endif

namespace dscuda {
namespace index_math {

// ---- LDS chunk permutations -------------------------------------------------
// A row-major LDS tile keeps 16-byte chunk c of row r at position c ^ f(r).
// Row bytes = 0 (mod 256): the four bits of the row, pairs exchanged.
// Row bytes = 128 (mod 256): the three bits of row>>1, bits 0 and 2 exchanged.
template <int ROW_BYTES>
DSCUDA_HOST_DEVICE constexpr int tile_swizzle(int row) {
    if constexpr (ROW_BYTES % 256 == 0) {
        return ((row & 3) << 2) | ((row >> 2) & 3);
    } else {
        const int u = row >> 1;
        return ((u & 1) << 2) | (u & 2) | ((u >> 2) & 1);
    }
}

// ---- backward workspace -----------------------------------------------------
// Position of dS block (key block kb of 128 keys, query tile qt of 64 queries),
// qt >= 2*kb, key block major; and the number of such blocks of one head.
DSCUDA_HOST_DEVICE inline long long ds_block_index(int kb, int qt, int query_tiles) {
    return (long long)kb * query_tiles - (long long)kb * (kb - 1) + (qt - 2 * kb);
}

DSCUDA_HOST_DEVICE inline long long ds_block_count(int key_blocks, int query_tiles) {
    return (long long)key_blocks * query_tiles - (long long)key_blocks * (key_blocks - 1);
}

// ---- tile requests of the backward kernels ------------------------------------
// One wave's share of the global -> LDS requests of a [ROWS][ROW_BYTES] tile that
// WAVES waves fetch together.  LDS slot 64*load + lane (16 bytes each) holds chunk
// (slot % CHUNKS) ^ f(row) of row slot / CHUNKS.  PERIOD loads cover PERIOD_ROWS
// whole rows; from one period to the next only the low bits of f change, so load
// L = PERIOD*m + r reads at
//     tile + m * PERIOD_ROWS * row_stride  +  (offset of load r) ^ 16 * (m % XOR_STEPS)
// The periods of a wave's LOADS consecutive loads are m = wave * LOADS/PERIOD + j;
// LOADS/PERIOD and XOR_STEPS are powers of two, so the two parts of m touch
// different bits of the XOR term: the wave's part is folded into a per-lane base
// once and j's part is a compile-time constant.
template <int ROW_BYTES, int WAVES, int ROWS = 64>
struct TileRequestMath {
    static constexpr int CHUNKS = ROW_BYTES / 16;
    static constexpr int LOADS = ROWS * ROW_BYTES / 1024 / WAVES;
    static constexpr int PERIOD = CHUNKS == 24 ? 3 : 1;
    static constexpr int PERIOD_ROWS = 64 * PERIOD / CHUNKS;
    static constexpr int XOR_STEPS = CHUNKS == 16 ? 4 : 2;
    static constexpr int PERIODS = LOADS / PERIOD;   // per wave
    static_assert(CHUNKS == 8 || CHUNKS == 16 || CHUNKS == 24, "rows of 128, 256 or 384 bytes");
    static_assert(ROWS * ROW_BYTES % (1024 * WAVES) == 0 && LOADS % PERIOD == 0, "tile must divide evenly over the waves");
    static_assert(PERIODS == 1 || PERIODS == 2 || PERIODS == 4, "periods per wave must be a power of two");

    // general form: byte offset of lane `lane` of load `load` from the tile's first row; rows past
    // `row_limit` repeat that row
    DSCUDA_HOST_DEVICE static unsigned offset_of(int load, int lane, unsigned row_stride, int row_limit) {
        const int slot = 64 * load + lane;
        const int row = slot / CHUNKS;
        const int chunk = (slot % CHUNKS) ^ tile_swizzle<ROW_BYTES>(row);
        return (unsigned)(row_limit < row ? row_limit : row) * row_stride + 16u * chunk;
    }
    // fast form, full tiles only: per-lane base of residue r (computed once per kernel) ...
    DSCUDA_HOST_DEVICE static unsigned base_of(int r, int lane, unsigned row_stride, int wave) {
        return offset_of(r, lane, row_stride, ROWS) ^ (16u * ((wave * PERIODS) % XOR_STEPS));
    }
    // ... the rows (from the tile's first) the uniform part of the address of the wave's load i skips ...
    DSCUDA_HOST_DEVICE static constexpr int rows_before(int i, int wave) {
        return wave * PERIODS * PERIOD_ROWS + i / PERIOD * PERIOD_ROWS;
    }
    // ... and the per-lane part of that load
    DSCUDA_HOST_DEVICE static constexpr unsigned lane_part(unsigned base, int i) {
        return base ^ (16u * ((i / PERIOD) % XOR_STEPS));
    }
};

// ---- fragment reads of the backward kernels ------------------------------------
// Per-lane byte offsets of the MFMA operand fragments inside a row-major swizzled
// LDS tile.  The swizzle only touches the low SPAN chunk positions of a row, so a
// handful of per-lane values plus compile-time constants reach every fragment.
//
//   natural(i, lane)        row lane%32, chunk (2i + g) ^ f(row), g = lane/32: the
//                           operand whose contraction index is the tile column;
//                           k-step ks = NAT*m + i lies NAT*32*m bytes further, 32
//                           rows down 32*ROW_BYTES (natural_constant)
//   transposed(h, i, lane)  for ds_read_b64_tr_b16: row 4g + s/4 + 8h (s = lane%16),
//                           chunk (4i + 2*((lane/16)%2) + (s%4)/2) ^ f(row), byte
//                           8*(s%2): the operand whose contraction index is the
//                           tile row; MFMA row/column lane%32 = tile column
//                           32*block + lane%32, k = rows {4g..4g+3, 8+4g..8+4g+3}
//                           of a 16-row step -- the order a C-layout register block
//                           carries; block = TR*m + i lies TR*64*m bytes further
//                           (transposed_constant)
//   quadrant(i, lane)       for the 16x16x32 products: row lane%16, chunk (4i + lane/16) ^ f(row):
//                           the operand whose contraction index is the tile column, 32 columns
//                           per step; step s = TR*m + i lies TR*64*m bytes further, 16 rows down
//                           16*ROW_BYTES (quadrant_constant; f repeats after 16 rows)
template <int ROW_BYTES>
struct TileReadMath {
    static constexpr int SPAN = (ROW_BYTES % 256 == 0) ? 16 : 8;
    static constexpr int NAT = SPAN / 2;
    static constexpr int TR = SPAN / 4;

    DSCUDA_HOST_DEVICE static unsigned natural(int i, int lane) {
        const int lq = lane % 32;
        const int g = lane / 32;
        return lq * ROW_BYTES + 16 * ((2 * i + g) ^ tile_swizzle<ROW_BYTES>(lq));
    }
    DSCUDA_HOST_DEVICE static unsigned transposed(int h, int i, int lane) {
        const int g = lane / 32;
        const int s = lane % 16;
        const int low = 2 * ((lane / 16) % 2) + (s % 4) / 2;
        const int row = 4 * g + s / 4 + 8 * h;
        return row * ROW_BYTES + 16 * ((4 * i + low) ^ tile_swizzle<ROW_BYTES>(row)) + 8 * (s % 2);
    }
    DSCUDA_HOST_DEVICE static unsigned quadrant(int i, int lane) {
        const int row = lane % 16;
        return row * ROW_BYTES + 16 * ((4 * i + lane / 16) ^ tile_swizzle<ROW_BYTES>(row));
    }
    DSCUDA_HOST_DEVICE static constexpr int quadrant_constant(int row0, int s) {
        return row0 * ROW_BYTES + (s / TR) * (TR * 64);
    }
    DSCUDA_HOST_DEVICE static constexpr int natural_constant(int row0, int ks) {
        return row0 * ROW_BYTES + (ks / NAT) * (NAT * 32);
    }
    DSCUDA_HOST_DEVICE static constexpr int transposed_constant(int row0, int block) {
        return row0 * ROW_BYTES + (block / TR) * (TR * 64);
    }
};

// ---- work order of the persistent forward kernel ------------------------------
struct ForwardItem {
    int batch_head;
    int query_block;
};

// Item `round` of workgroup `member` (of `members`) of a cluster that owns
// `cluster_heads` (batch, head) pairs (pairs cluster, cluster + clusters, ...);
// false past the end of the list.  Inside a cluster the items are laid out two
// heads at a time (one if the count is odd), blocks from the heaviest (last) to
// the lightest, and cut into rounds of one item per workgroup; odd rounds are
// handed out in reverse.
DSCUDA_HOST_DEVICE inline bool forward_item(int round, int member, int members, int cluster, int clusters,
                                            int cluster_heads, int query_blocks, ForwardItem& item) {
    const int position = (round & 1) ? members - 1 - member : member;
    const int index = round * members + position;
    if (index >= cluster_heads * query_blocks) {
        return false;
    }
    const int interleave = (cluster_heads % 2 == 0) ? 2 : 1;
    const int group = index / (interleave * query_blocks);
    const int rest = index % (interleave * query_blocks);
    item.batch_head = cluster + clusters * (interleave * group + rest % interleave);
    item.query_block = query_blocks - 1 - rest / interleave;
    return true;
}

// ---- decode: tile loads -------------------------------------------------------
// A [4 * ROWS_PER_WAVE][ROW_BYTES] tile of consecutive rows is fetched by four waves,
// wave w filling rows ROWS_PER_WAVE*w .. +ROWS_PER_WAVE-1 with 1 KB instructions: LDS
// slot 64*i + lane of the wave's share (16 bytes each) holds chunk (slot % CHUNKS) ^
// f(row) of local row slot / CHUNKS.  With i a compile-time constant a wave
// instruction spans at most two rows, so the row part of the offset is wave-uniform
// and the lane part costs an add, an xor and a shift-add per candidate row.  Rows
// past `row_limit` (of the tile) repeat that row.  ROWS_PER_WAVE = 16 is the 64-key
// tile, 8 the 32-key unit.
template <int ROW_BYTES, int ROWS_PER_WAVE = 16>
DSCUDA_HOST_DEVICE inline unsigned contiguous_load_offset(int wave, int i, int lane, int row_limit) {
    constexpr int CHUNKS = ROW_BYTES / 16;
    const int first_row = (64 * i) / CHUNKS;                 // row of lane 0 (within the wave's rows)
    const int boundary = CHUNKS * (first_row + 1) - 64 * i;  // first lane of the next row (may be >= 64)
    const int tile_row_a = ROWS_PER_WAVE * wave + first_row;
    const unsigned row_a = (unsigned)(tile_row_a < row_limit ? tile_row_a : row_limit) * ROW_BYTES;
    unsigned offset = row_a + 16u * (unsigned)((lane + 64 * i - CHUNKS * first_row) ^ tile_swizzle<ROW_BYTES>(tile_row_a));
    if (boundary < 64) {
        const int tile_row_b = tile_row_a + 1;
        const unsigned row_b = (unsigned)(tile_row_b < row_limit ? tile_row_b : row_limit) * ROW_BYTES;
        const unsigned other =
            row_b + 16u * (unsigned)((lane + 64 * i - CHUNKS * (first_row + 1)) ^ tile_swizzle<ROW_BYTES>(tile_row_b));
        offset = lane >= boundary ? other : offset;
    }
    return offset;
}

// ---- decode: cutting the work list ---------------------------------------------
// Every sequence with tokens contributes `overhead` + tiles positions to one list
// (sequence after sequence): its 64-token tiles, preceded by positions that stand for
// what a workgroup spends on a segment besides its tiles (query rows, the first
// requests, filling and draining the pipeline, storing the result), so that ranges of
// equal length take about equal time.  The list is cut into W = min(workgroups, total)
// ranges, none empty, whose lengths differ by at most one: range w is
// [w * total / W, (w + 1) * total / W).  A
// range computes the tiles whose positions it holds; a range that holds only part of
// the tiles of a sequence leaves a partial result in slot workgroup + sequence: ranges
// and sequences both advance monotonically, so no two (range, sequence) pairs that
// intersect share a slot, and every slot is below workgroups + sequences.
constexpr int SEGMENT_OVERHEAD = 6;   // in tiles: what a segment costs before, between and after its tiles

DSCUDA_HOST_DEVICE inline int positions_of(int tiles, int overhead) { return tiles > 0 ? tiles + overhead : 0; }

DSCUDA_HOST_DEVICE inline int ranges_of(int total, int workgroups) { return total < workgroups ? total : workgroups; }

// First position of range `range` (0 .. ranges: the last one is the end of the list).
DSCUDA_HOST_DEVICE inline int range_begin_of(int total, int ranges, int range) {
    return (int)((long long)range * total / ranges);
}

// The range that holds position `position` (0 <= position < total).
DSCUDA_HOST_DEVICE inline int range_of_position(int total, int ranges, int position) {
    return (int)((((long long)position + 1) * ranges - 1) / total);
}

// Tiles [first, last) that the positions [begin, end) hold of a sequence whose positions
// start at `before`; last <= first when they hold none.
DSCUDA_HOST_DEVICE inline void tiles_in_positions(int begin, int end, int before, int overhead, int& first, int& last) {
    const int low = begin - before - overhead;
    const int high = end - before - overhead;
    first = low > 0 ? low : 0;
    last = high > 0 ? high : 0;
}

// First and last range that hold tiles of a sequence of `positions` > 0 positions that starts at `before`.
DSCUDA_HOST_DEVICE inline void ranges_of_sequence(int total, int ranges, int before, int positions, int overhead,
                                                  int& first, int& last) {
    first = range_of_position(total, ranges, before + overhead);
    last = range_of_position(total, ranges, before + positions - 1);
}

// ---- absorbed backward: the list of (key block, row tile) visits -----------------
// Rows are the (token, head) pairs of one batch element in memory order, 32 to a row
// tile (`row_tiles` of them); key block kb (32 keys) is seen by the row tiles from
// kb * heads (the tile of row 32 * kb * heads, the first row of token 32 * kb) to the
// last.  The visits of all key blocks of all batch elements, in that order, form one
// list that the key-gradient kernel cuts into ranges of equal length (+-1); a range
// that holds only part of a key block's visits leaves an fp32 partial result in slot
// range + (batch * key_blocks + key block): ranges and key blocks both advance
// monotonically along the list, so the sums are distinct and below ranges + blocks.
struct KeyVisits {
    int key_blocks;
    int row_tiles;
    int heads;

    DSCUDA_HOST_DEVICE long long before(int key_block) const {   // visits of key blocks 0 .. key_block-1
        return (long long)key_block * row_tiles - (long long)heads * key_block * (key_block - 1) / 2;
    }
    DSCUDA_HOST_DEVICE long long per_batch() const { return before(key_blocks); }
    DSCUDA_HOST_DEVICE int first_tile(int key_block) const { return key_block * heads; }
    // the key block that holds visit `visit` (0 <= visit < per_batch())
    DSCUDA_HOST_DEVICE int block_of(long long visit) const {
        int low = 0, high = key_blocks - 1;
        while (low < high) {
            const int middle = (low + high + 1) / 2;
            if (before(middle) <= visit) low = middle; else high = middle - 1;
        }
        return low;
    }
};

// `key_tiles`: key blocks of 32 * key_tiles keys.  Such a block is seen from the tile of row 32 * key_tiles * kb * heads
// on, which is what blocks of 32 keys and key_tiles * heads heads give: `heads` holds that product.
DSCUDA_HOST_DEVICE inline KeyVisits key_visits(int sequence_length, int heads, int key_tiles = 1) {
    KeyVisits visits;
    visits.key_blocks = (sequence_length + 32 * key_tiles - 1) / (32 * key_tiles);
    visits.row_tiles = (int)(((long long)sequence_length * heads + 31) / 32);
    visits.heads = heads * key_tiles;
    return visits;
}

DSCUDA_HOST_DEVICE inline long long wide_range_begin(long long total, long long ranges, long long range) {
    return range * total / ranges;
}

DSCUDA_HOST_DEVICE inline long long wide_range_of(long long total, long long ranges, long long position) {
    return ((position + 1) * ranges - 1) / total;
}

// Large inputs (the query and dO rows of a batch element no longer stay in the caches): equal ranges would have
// every workgroup stream its own stretch of rows from memory, one pass over all rows per key block.  Instead the
// row tiles are cut into intervals of `length` tiles and the work into items (interval, key block), numbered
// interval by interval, so that the workgroups running at any time walk the same few intervals and all but
// the first of them find the rows in the caches.  Item (i, kb) exists when the block sees the interval
// (kb * heads < end of interval i), covers the block's tiles inside it, and leaves its partial result in the
// slot of its own number (none when it is the block's only item, i.e. the block starts in the last interval).
struct KeyIntervals {
    int length;      // row tiles per interval
    int intervals;
    int heads;
    int key_blocks;
    int row_tiles;

    DSCUDA_HOST_DEVICE int end_of(int interval) const {
        const long long end = (long long)(interval + 1) * length;
        return end < row_tiles ? (int)end : row_tiles;
    }
    DSCUDA_HOST_DEVICE int blocks_in(int interval) const {   // key blocks 0 .. blocks_in-1 see the interval
        const int seen = (end_of(interval) + heads - 1) / heads;
        return seen < key_blocks ? seen : key_blocks;
    }
    DSCUDA_HOST_DEVICE long long items_before(int interval) const {
        long long items = 0;
        for (int i = 0; i < interval; ++i) items += blocks_in(i);
        return items;
    }
    DSCUDA_HOST_DEVICE long long items() const { return items_before(intervals); }
    DSCUDA_HOST_DEVICE int first_interval(int key_block) const { return (int)((long long)key_block * heads / length); }
    // item number (within its batch element) -> interval, key block
    DSCUDA_HOST_DEVICE void locate(long long item, int& interval, int& key_block) const {
        interval = 0;
        while (item >= blocks_in(interval)) {
            item -= blocks_in(interval);
            ++interval;
        }
        key_block = (int)item;
    }
};

DSCUDA_HOST_DEVICE inline KeyIntervals key_intervals(int sequence_length, int heads, int length, int key_tiles = 1) {
    KeyIntervals cut;
    cut.length = length;
    cut.heads = heads * key_tiles;   // as in key_visits
    cut.key_blocks = (sequence_length + 32 * key_tiles - 1) / (32 * key_tiles);
    cut.row_tiles = (int)(((long long)sequence_length * heads + 31) / 32);
    cut.intervals = (cut.row_tiles + length - 1) / length;
    return cut;
}

constexpr long long KEY_PARTIAL_BYTES = 32LL * 576 * 4;   // one slot: [32 keys][576] fp32

// Interval length (row tiles) of the cut into items: the shortest of the ladder 24, 32, 48, 64, 96, ... whose items,
// over `batch` batch elements, number at most twelve rounds of the compute units and have a slot each (shorter
// intervals give more, shorter items: a fuller last round, as long as the slots last).  0: even that many items
// are fewer than two rounds, or no length of the ladder fits; equal ranges balance the units better then.
DSCUDA_HOST_DEVICE inline int key_interval_choice(int sequence_length, int heads, long long batch, long long slots,
                                                  int compute_units, int key_tiles) {
    const long long rounds = 12LL * compute_units;
    const long long most = rounds < slots ? rounds : slots;
    const long long row_tiles = ((long long)sequence_length * heads + 31) / 32;
    for (long long base = 8; ; base *= 2) {
        for (int multiple = 3; multiple <= 4; ++multiple) {
            const long long tiles = base * multiple;
            if (tiles >= (1 << 24)) return 0;
            const long long items = key_intervals(sequence_length, heads, (int)tiles, key_tiles).items() * batch;
            if (items <= most) return items >= 2LL * compute_units ? (int)tiles : 0;
            if (tiles >= row_tiles) return 0;
        }
    }
}

// How many ranges the list is cut into when `scratch_bytes` are there for the slots: one per compute unit if the
// slots allow.  0: every key block is one range and writes its result itself (too few slots for a cut whose
// longest range is shorter than the longest key block, `row_tiles` visits).
DSCUDA_HOST_DEVICE inline long long key_gradient_ranges(long long total, long long blocks, int row_tiles,
                                                        long long scratch_bytes, int compute_units) {
    const long long slots = scratch_bytes / KEY_PARTIAL_BYTES;
    long long ranges = slots - blocks;
    if (ranges > compute_units) ranges = compute_units;
    if (ranges > total / 2) ranges = total / 2;    // at least two visits per range
    if (ranges < 2) return 0;
    const long long longest = (total + ranges - 1) / ranges;
    return (longest < row_tiles || blocks > compute_units) ? ranges : 0;
}

// ---- decode: the plan and how a call uses the caller's workspace ---------------
// The plan is what a decode call needs to know about the lengths of its batch
// before any workgroup starts: an int table
//     [0] total positions   [1] workgroups   [2] overhead positions per sequence   [3] 1 = sequences are not cut
//     [4] ranges the list is cut into (<= workgroups)
//     [5 .. 5+B]        inclusive prefix of positions per sequence (B + 1 entries)
//     [.. + W]          first sequence whose positions reach past the start of each range
// It is read-only once built.
constexpr int PLAN_TOTAL = 0;
constexpr int PLAN_WORKGROUPS = 1;
constexpr int PLAN_OVERHEAD = 2;
constexpr int PLAN_WHOLE = 3;
constexpr int PLAN_RANGES = 4;
constexpr int PLAN_HEADER = 5;

DSCUDA_HOST_DEVICE inline long long plan_prefix_at() { return PLAN_HEADER; }
DSCUDA_HOST_DEVICE inline long long plan_first_sequence_at(int batch) { return PLAN_HEADER + (long long)batch + 1; }
DSCUDA_HOST_DEVICE inline long long plan_elements(int batch, int workgroups) {
    return plan_first_sequence_at(batch) + workgroups;
}
// Size of a plan buffer that fits whatever device builds the plan: a call cuts its list into at
// most one range per compute unit (the host clamps the count it asks the device for to
// PLAN_MAX_WORKGROUPS), or runs one workgroup per sequence.
constexpr int PLAN_MAX_WORKGROUPS = 1024;
DSCUDA_HOST_DEVICE inline long long plan_elements_bound(int batch) {
    return plan_elements(batch, batch > PLAN_MAX_WORKGROUPS ? batch : PLAN_MAX_WORKGROUPS);
}

// The caller's workspace holds batch * heads * splits * (rank + 2) floats.  A
// range that holds only part of a sequence leaves its unnormalised result there:
// slot workgroup + sequence (slots = workgroups + batch), each slot one bf16 row of
// `rank` values plus two floats (reference exponent, sum) per head, heads rounded up
// to whole waves of 32.  A call without a caller-provided plan keeps its plan behind
// the slots.  The number of workgroups is the largest (up to one per compute unit)
// for which all of that fits; when fewer than two fit, no sequence is cut: one
// workgroup per sequence, no slots.
struct DecodeLayout {
    int workgroups;
    int whole_sequences;
    int head_groups;
    long long slot_floats;
    long long slots;
    long long plan_offset;   // in floats from the start of the workspace
    long long plan_ints;
};

DSCUDA_HOST_DEVICE inline DecodeLayout decode_layout(int batch, int heads, int splits, int compute_units,
                                                     int rows_per_group, int rank) {
    DecodeLayout layout;
    layout.head_groups = (heads + rows_per_group - 1) / rows_per_group;
    const long long padded_rows = (long long)((heads + 31) / 32) * 32;
    layout.slot_floats = padded_rows * (rank / 2 + 2);
    const long long workspace = (long long)batch * heads * splits * (rank + 2);
    // (W + batch) * slot_floats + plan_elements(batch, W) <= workspace, W <= compute_units
    const long long fixed = (long long)batch * layout.slot_floats + plan_elements(batch, 0);
    long long cutting = workspace >= fixed ? (workspace - fixed) / (layout.slot_floats + 1) : 0;
    if (cutting > compute_units) cutting = compute_units;
    layout.whole_sequences = (splits <= 1 || cutting < 2) ? 1 : 0;
    if (layout.whole_sequences) {
        layout.workgroups = batch;
        layout.slots = 0;
    } else {
        layout.workgroups = (int)cutting;
        layout.slots = (long long)layout.workgroups + batch;
    }
    layout.plan_offset = layout.slots * layout.slot_floats;
    layout.plan_ints = plan_elements(batch, layout.workgroups);
    return layout;
}

}  // namespace index_math
}  // namespace dscuda
