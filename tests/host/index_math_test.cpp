// Exhaustive host-side checks of dscuda_amd/csrc/index_math.h, the integer arithmetic the kernels share with
// this test: compiled with the host compiler and run by tests/test_index_math.py.  Every check enumerates its
// whole domain; a failure prints the first counterexample and the program exits non-zero.
#include "index_math.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <set>
#include <utility>
#include <vector>

using namespace dscuda::index_math;

static int failures = 0;
#define EXPECT(condition, ...)                                  \
    do {                                                        \
        if (!(condition)) {                                     \
            if (failures++ < 20) {                              \
                std::printf("FAIL %s:%d %s: ", __FILE__, __LINE__, #condition); \
                std::printf(__VA_ARGS__);                       \
                std::printf("\n");                              \
            }                                                   \
        }                                                       \
    } while (0)

// ---- chunk permutation: stays inside the row, is a permutation, and spreads the two read patterns over the banks
template <int ROW_BYTES>
void check_swizzle() {
    constexpr int CHUNKS = ROW_BYTES / 16;
    constexpr int SPAN = ROW_BYTES % 256 == 0 ? 16 : 8;
    for (int row = 0; row < 128; ++row) {
        const int f = tile_swizzle<ROW_BYTES>(row);
        EXPECT(f >= 0 && f < SPAN, "ROW_BYTES %d row %d f %d", ROW_BYTES, row, f);
        std::set<int> seen;
        for (int chunk = 0; chunk < CHUNKS; ++chunk) {
            const int position = chunk ^ f;
            EXPECT(position >= 0 && position < CHUNKS, "ROW_BYTES %d row %d chunk %d -> %d", ROW_BYTES, row, chunk, position);
            seen.insert(position);
        }
        EXPECT((int)seen.size() == CHUNKS, "ROW_BYTES %d row %d not a permutation", ROW_BYTES, row);
    }
    // 16-byte reads down a column: 16 lanes (rows r0 .. r0+15, the same chunk c of each) are served together and
    // must touch 16 different 16-byte bank groups of the 256-byte bank line
    for (int r0 = 0; r0 < 64; r0 += 16) {
        for (int chunk = 0; chunk < CHUNKS; ++chunk) {
            std::set<int> groups;
            for (int lane = 0; lane < 16; ++lane) {
                const int row = r0 + lane;
                const int address = row * ROW_BYTES + 16 * (chunk ^ tile_swizzle<ROW_BYTES>(row));
                groups.insert(address / 16 % 16);
            }
            EXPECT(groups.size() == 16, "ROW_BYTES %d rows %d.. chunk %d: %zu of 16 bank groups", ROW_BYTES, r0, chunk, groups.size());
        }
    }
    // transposing 8-byte reads: 16 lanes cover 4 rows (r0 .. r0+3, r0 a multiple of 4) x one 64-byte column block
    // (chunks 4b .. 4b+3, two lanes per chunk): the 16 chunks touched must lie in 16 different bank groups
    for (int r0 = 0; r0 < 64; r0 += 4) {
        for (int block = 0; block < CHUNKS / 4; ++block) {
            std::set<int> groups;
            for (int row = r0; row < r0 + 4; ++row) {
                for (int c = 0; c < 4; ++c) {
                    const int address = row * ROW_BYTES + 16 * ((4 * block + c) ^ tile_swizzle<ROW_BYTES>(row));
                    groups.insert(address / 16 % 16);
                }
            }
            EXPECT(groups.size() == 16, "ROW_BYTES %d rows %d.. block %d: %zu of 16 bank groups", ROW_BYTES, r0, block, groups.size());
        }
    }
}

// ---- tile requests: the fast form equals the general form, and the loads of all waves tile the LDS copy exactly
template <int ROW_BYTES, int WAVES>
void check_requests() {
    using Math = TileRequestMath<ROW_BYTES, WAVES, 64>;
    for (unsigned heads : {1u, 3u, 128u}) {
        const unsigned row_stride = heads * ROW_BYTES;
        std::vector<int> covered(64 * Math::CHUNKS, 0);
        for (int wave = 0; wave < WAVES; ++wave) {
            for (int i = 0; i < Math::LOADS; ++i) {
                for (int lane = 0; lane < 64; ++lane) {
                    const int load = wave * Math::LOADS + i;
                    const unsigned general = Math::offset_of(load, lane, row_stride, 63);
                    const unsigned base = Math::base_of(i % Math::PERIOD, lane, row_stride, wave);
                    const unsigned long long fast = (unsigned long long)Math::rows_before(i, wave) * row_stride + Math::lane_part(base, i);
                    EXPECT(fast == general, "ROW_BYTES %d WAVES %d stride %u wave %d load %d lane %d: fast %llu general %u",
                           ROW_BYTES, WAVES, row_stride, wave, i, lane, fast, general);
                    // LDS slot 64*load + lane must receive chunk (slot % CHUNKS) ^ f(row) of row slot / CHUNKS
                    const int slot = 64 * load + lane;
                    const int row = slot / Math::CHUNKS;
                    const unsigned expected = (unsigned)row * row_stride + 16u * ((slot % Math::CHUNKS) ^ tile_swizzle<ROW_BYTES>(row));
                    EXPECT(general == expected, "slot %d", slot);
                    const int source_chunk = (int)((general - (unsigned)row * row_stride) / 16);
                    ++covered[row * Math::CHUNKS + source_chunk];
                }
            }
        }
        for (int index = 0; index < 64 * Math::CHUNKS; ++index) {
            EXPECT(covered[index] == 1, "ROW_BYTES %d WAVES %d: chunk %d of the tile fetched %d times", ROW_BYTES, WAVES, index, covered[index]);
        }
        // ragged end: rows past the limit repeat the limit row, nothing before the tile or past that row is read
        for (int row_limit : {0, 1, 17, 62}) {
            for (int load = 0; load < WAVES * Math::LOADS; ++load) {
                for (int lane = 0; lane < 64; ++lane) {
                    const unsigned offset = Math::offset_of(load, lane, row_stride, row_limit);
                    EXPECT(offset < (unsigned)row_limit * row_stride + ROW_BYTES, "row_limit %d load %d lane %d offset %u", row_limit, load, lane, offset);
                }
            }
        }
    }
}

// ---- fragment reads: which tile element ends up in which operand register
// A byte address inside a swizzled LDS tile -> (row, first column) of the 16-bit elements stored there.
template <int ROW_BYTES>
void locate(unsigned address, int& row, int& column) {
    row = (int)(address / ROW_BYTES);
    const int in_row = (int)(address % ROW_BYTES);
    const int chunk = (in_row / 16) ^ tile_swizzle<ROW_BYTES>(row);
    column = 8 * chunk + (in_row % 16) / 2;
}

// MFMA 32x32x16 operand layout: lane l holds row (or column) l % 32 of the operand and the eight contraction
// indices 8 * (l / 32) + j.  ds_read_b64_tr_b16: within a block of 16 lanes, lane i receives, as element e of its
// four, 16-bit element i % 4 of the eight bytes that lane i / 4 + 4 * e addressed.
template <int ROW_BYTES>
void check_fragment_reads() {
    using Math = TileReadMath<ROW_BYTES>;
    constexpr int COLUMNS = ROW_BYTES / 2;
    // natural: operand row = tile row ROW0 + l % 32, contraction index = tile column 16 * KS + 8 * (l / 32) + j
    for (int row0 : {0, 32}) {
        for (int ks = 0; ks < COLUMNS / 16; ++ks) {
            for (int lane = 0; lane < 64; ++lane) {
                int row, column;
                locate<ROW_BYTES>(Math::natural(ks % Math::NAT, lane) + Math::natural_constant(row0, ks), row, column);
                EXPECT(row == row0 + lane % 32 && column == 16 * ks + 8 * (lane / 32),
                       "natural ROW_BYTES %d row0 %d ks %d lane %d -> row %d column %d", ROW_BYTES, row0, ks, lane, row, column);
            }
        }
    }
    // quadrant (16x16x32 operand layout: lane l holds row l % 16 and contraction indices 8 * (l / 16) + j of a
    // 32-column step): operand row = tile row ROW0 + l % 16, first column 32 * S + 8 * (l / 16)
    for (int row0 : {0, 16, 32, 48}) {
        for (int step = 0; step < COLUMNS / 32; ++step) {
            for (int lane = 0; lane < 64; ++lane) {
                int row, column;
                locate<ROW_BYTES>(Math::quadrant(step % Math::TR, lane) + Math::quadrant_constant(row0, step), row, column);
                EXPECT(row == row0 + lane % 16 && column == 32 * step + 8 * (lane / 16),
                       "quadrant ROW_BYTES %d row0 %d step %d lane %d -> row %d column %d", ROW_BYTES, row0, step, lane, row, column);
            }
        }
    }
    // transposed: operand row = tile column 32 * BLOCK + l % 32, contraction index j -> tile row
    // ROW0 + {4g .. 4g+3, 8+4g .. 8+4g+3}[j], g = l / 32 (two reads, h = 0 for j < 4, h = 1 for j >= 4)
    for (int row0 : {0, 16, 32, 48}) {
        for (int block = 0; block < COLUMNS / 32; ++block) {
            for (int h = 0; h < 2; ++h) {
                unsigned address[64];
                for (int lane = 0; lane < 64; ++lane) {
                    address[lane] = Math::transposed(h, block % Math::TR, lane) + Math::transposed_constant(row0, block);
                    EXPECT(address[lane] % 8 == 0, "transposed read not 8-byte aligned");
                }
                for (int lane = 0; lane < 64; ++lane) {
                    const int block16 = lane / 16, i = lane % 16, g = lane / 32;
                    for (int e = 0; e < 4; ++e) {
                        const int source = 16 * block16 + i / 4 + 4 * e;
                        int row, column;
                        locate<ROW_BYTES>(address[source], row, column);
                        column += i % 4;
                        EXPECT(column == 32 * block + lane % 32 && row == row0 + 8 * h + 4 * g + e,
                               "transposed ROW_BYTES %d row0 %d block %d h %d lane %d e %d -> row %d column %d", ROW_BYTES, row0,
                               block, h, lane, e, row, column);
                    }
                }
            }
        }
    }
}

// ---- dS blocks: key-block-major enumeration of the causal (key block, query tile) pairs, without gaps
void check_ds_blocks() {
    for (int sequence = 1; sequence <= 4200; sequence += (sequence < 600 ? 1 : 97)) {
        const int query_tiles = (sequence + 63) / 64, key_blocks = (sequence + 127) / 128;
        long long next = 0;
        for (int kb = 0; kb < key_blocks; ++kb) {
            for (int qt = 2 * kb; qt < query_tiles; ++qt) {
                EXPECT(ds_block_index(kb, qt, query_tiles) == next, "S %d kb %d qt %d", sequence, kb, qt);
                ++next;
            }
        }
        EXPECT(ds_block_count(key_blocks, query_tiles) == next, "S %d count %lld enumerated %lld", sequence,
               ds_block_count(key_blocks, query_tiles), next);
    }
}

// ---- forward work order: every (batch*head, query block) exactly once, heads stay with their cluster, and with an
// even number of heads per cluster and rounds that divide evenly every workgroup gets the same number of key tiles
void check_forward_items() {
    for (int clusters : {1, 8}) {
        for (int batch_heads : {1, 2, 7, 8, 16, 24, 40, 128, 136}) {
            if (batch_heads % clusters != 0) continue;
            for (int query_blocks : {1, 2, 3, 5, 16, 64}) {
                const int cluster_heads = batch_heads / clusters;
                for (int members : {1, 2, 3, 5, 32}) {
                    if (members > cluster_heads * query_blocks) continue;
                    std::vector<int> visits(batch_heads * query_blocks, 0);
                    long long lightest = -1, heaviest = -1;
                    for (int cluster = 0; cluster < clusters; ++cluster) {
                        for (int member = 0; member < members; ++member) {
                            long long work = 0;
                            ForwardItem item;
                            int round = 0;
                            for (; forward_item(round, member, members, cluster, clusters, cluster_heads, query_blocks, item); ++round) {
                                EXPECT(item.batch_head >= 0 && item.batch_head < batch_heads && item.batch_head % clusters == cluster,
                                       "head %d cluster %d", item.batch_head, cluster);
                                EXPECT(item.query_block >= 0 && item.query_block < query_blocks, "block %d", item.query_block);
                                ++visits[item.batch_head * query_blocks + item.query_block];
                                work += item.query_block + 1;
                            }
                            // the list ends for good: no item reappears after the first miss
                            EXPECT(!forward_item(round + 1, member, members, cluster, clusters, cluster_heads, query_blocks, item) ||
                                       round * members + members > cluster_heads * query_blocks - members,
                                   "item after the end");
                            lightest = lightest < 0 ? work : std::min(lightest, work);
                            heaviest = std::max(heaviest, work);
                        }
                    }
                    for (int index = 0; index < batch_heads * query_blocks; ++index) {
                        EXPECT(visits[index] == 1, "clusters %d heads %d blocks %d members %d: item %d visited %d times", clusters,
                               batch_heads, query_blocks, members, index, visits[index]);
                    }
                    const int rounds = cluster_heads * query_blocks / members;
                    if (cluster_heads % 2 == 0 && (cluster_heads * query_blocks) % members == 0 && rounds % 2 == 0 &&
                        (2 * query_blocks) % members == 0) {
                        EXPECT(lightest == heaviest, "clusters %d heads %d blocks %d members %d: work %lld .. %lld", clusters, batch_heads,
                               query_blocks, members, lightest, heaviest);
                    }
                }
            }
        }
    }
}

// ---- decode tile loads: the two-candidate-row form equals the general form for every wave, load, lane and limit,
// for the 64-key tile (16 rows per wave, 18 loads), the 32-key unit (8 rows per wave, 9 loads) and 32 rows per wave
template <int ROWS_PER_WAVE>
void check_decode_loads() {
    constexpr int ROW_BYTES = 1152, CHUNKS = ROW_BYTES / 16, LOADS = ROWS_PER_WAVE * CHUNKS / 64, ROWS = 4 * ROWS_PER_WAVE;
    for (int row_limit : {0, 1, 7, 8, 15, 16, 17, 31, 40, 62, 63, 64, 1000}) {
        std::vector<int> fetched(ROWS * CHUNKS, 0);
        for (int wave = 0; wave < 4; ++wave) {
            for (int i = 0; i < LOADS; ++i) {
                for (int lane = 0; lane < 64; ++lane) {
                    const int slot = 64 * i + lane;                  // of the wave's share
                    const int local_row = slot / CHUNKS, position = slot % CHUNKS;
                    const int row = ROWS_PER_WAVE * wave + local_row;
                    const int chunk = position ^ tile_swizzle<ROW_BYTES>(row);
                    const unsigned general = (unsigned)std::min(row, row_limit) * ROW_BYTES + 16u * chunk;
                    const unsigned fast = contiguous_load_offset<ROW_BYTES, ROWS_PER_WAVE>(wave, i, lane, row_limit);
                    EXPECT(fast == general, "rows/wave %d row_limit %d wave %d load %d lane %d: %u vs %u", ROWS_PER_WAVE, row_limit, wave, i,
                           lane, fast, general);
                    // nothing past the limit row is read
                    EXPECT(fast < (unsigned)std::min(row_limit, ROWS - 1) * ROW_BYTES + ROW_BYTES, "row_limit %d offset %u", row_limit, fast);
                    if (row_limit >= ROWS - 1) ++fetched[row * CHUNKS + chunk];
                }
            }
        }
        if (row_limit >= ROWS - 1) {
            for (int index = 0; index < ROWS * CHUNKS; ++index) EXPECT(fetched[index] == 1, "chunk %d fetched %d times", index, fetched[index]);
        }
    }
}

// ---- absorbed backward: the list of (key block, row tile) visits.  A row tile is visited by a key block exactly when
// one of its rows can see one of the block's keys; the closed forms agree with enumeration; the ranges partition the
// list; (range, block) pairs that hold part of a block own distinct slots below the slot count the cut was sized for.
void check_key_visits() {
    for (int heads : {1, 2, 3, 4, 8, 16, 20, 128}) {
        for (int tokens : {1, 5, 31, 32, 33, 96, 128, 257, 512, 1000}) {
            if ((long long)heads * tokens > 40000) continue;
            const KeyVisits visits = key_visits(tokens, heads);
            const long long rows = (long long)heads * tokens;
            EXPECT(visits.key_blocks == (tokens + 31) / 32 && visits.row_tiles == (rows + 31) / 32, "counts");
            long long before = 0;
            for (int kb = 0; kb < visits.key_blocks; ++kb) {
                EXPECT(visits.before(kb) == before, "heads %d tokens %d block %d: before %lld vs %lld", heads, tokens, kb, visits.before(kb), before);
                int first = -1, count = 0;
                for (int tile = 0; tile < visits.row_tiles; ++tile) {
                    const long long last_row = std::min<long long>(rows, 32LL * (tile + 1)) - 1;
                    if (last_row / heads >= 32 * kb) {   // the tile's last token sees the block's first key
                        if (first < 0) first = tile;
                        ++count;
                    }
                }
                EXPECT(count >= 1 && first == visits.first_tile(kb), "heads %d tokens %d block %d: first tile %d vs %d", heads, tokens, kb, first, visits.first_tile(kb));
                for (long long v = before; v < before + count; v += std::max(1, count / 7)) EXPECT(visits.block_of(v) == kb, "block_of");
                EXPECT(visits.block_of(before + count - 1) == kb, "block_of last");
                before += count;
            }
            EXPECT(visits.per_batch() == before, "per_batch");
            for (int batch : {1, 2, 3}) {
                const long long total = before * batch, blocks = (long long)visits.key_blocks * batch;
                for (int units : {4, 256}) {
                    for (long long scratch : {0LL, rows * batch * 1024, rows * batch * 1024 / 3, 1LL << 40}) {
                        const long long ranges = key_gradient_ranges(total, blocks, visits.row_tiles, scratch, units);
                        if (ranges == 0) continue;
                        EXPECT(ranges >= 2 && ranges <= units && ranges + blocks <= scratch / KEY_PARTIAL_BYTES && 2 * ranges <= total,
                               "ranges %lld blocks %lld scratch %lld", ranges, blocks, scratch);
                        std::set<long long> slots;
                        long long covered = 0;
                        for (long long r = 0; r < ranges; ++r) {
                            const long long begin = wide_range_begin(total, ranges, r), end = wide_range_begin(total, ranges, r + 1);
                            EXPECT(end > begin, "empty range");
                            EXPECT(wide_range_of(total, ranges, begin) == r && wide_range_of(total, ranges, end - 1) == r, "range_of");
                            long long position = begin;
                            while (position < end) {   // the kernel's walk
                                const int b = (int)(position / before);
                                const long long within = position - b * before;
                                const int kb = visits.block_of(within);
                                const long long segment_end = std::min(end - b * before, visits.before(kb + 1));
                                const bool whole = within == visits.before(kb) && segment_end == visits.before(kb + 1);
                                if (!whole) {
                                    const long long slot = r + (long long)b * visits.key_blocks + kb;
                                    EXPECT(slot < scratch / KEY_PARTIAL_BYTES, "slot %lld", slot);
                                    EXPECT(slots.insert(slot).second, "slot %lld used twice", slot);
                                    // the reduction finds it: the block's first range + offset
                                    const long long g_begin = b * before + visits.before(kb);
                                    const long long first_range = wide_range_of(total, ranges, g_begin);
                                    const long long last_range = wide_range_of(total, ranges, b * before + visits.before(kb + 1) - 1);
                                    EXPECT(first_range < last_range && r >= first_range && r <= last_range, "reduction range");
                                } else {
                                    const long long g_begin = b * before + visits.before(kb);
                                    EXPECT(wide_range_of(total, ranges, g_begin) == wide_range_of(total, ranges, b * before + visits.before(kb + 1) - 1), "whole block");
                                }
                                covered += segment_end - within;
                                position = b * before + segment_end;
                            }
                        }
                        EXPECT(covered == total, "covered %lld of %lld", covered, total);
                    }
                }
            }
        }
    }
}

// ---- absorbed backward, interval cut: the items cover every (key block, row tile) visit exactly once, item numbers
// are a bijection, a block has one item exactly when it starts in the last interval
void check_key_intervals() {
    for (int heads : {1, 3, 8, 16, 128}) {
        for (int tokens : {1, 33, 257, 512, 1000}) {
            if ((long long)heads * tokens > 70000) continue;
            for (int length : {1, 2, 7, 64, 100000}) for (int key_tiles : {1, 2}) {
                const KeyIntervals cut = key_intervals(tokens, heads, length, key_tiles);
                const KeyVisits visits = key_visits(tokens, heads, key_tiles);
                EXPECT(cut.key_blocks == visits.key_blocks && cut.row_tiles == visits.row_tiles, "counts");
                EXPECT(cut.key_blocks == (tokens + 32 * key_tiles - 1) / (32 * key_tiles), "key blocks");
                for (int kb = 0; kb < cut.key_blocks; ++kb) {
                    // the first tile that holds a row of the block's first token
                    EXPECT(visits.first_tile(kb) == (int)((long long)32 * key_tiles * kb * heads / 32), "first tile");
                }
                std::vector<int> seen((size_t)cut.key_blocks * cut.row_tiles, 0), parts(cut.key_blocks, 0);
                long long item = 0;
                for (int i = 0; i < cut.intervals; ++i) {
                    EXPECT(cut.items_before(i) == item, "items_before");
                    for (int kb = 0; kb < cut.blocks_in(i); ++kb, ++item) {
                        int interval, key_block;
                        cut.locate(item, interval, key_block);
                        EXPECT(interval == i && key_block == kb, "locate %lld: %d %d vs %d %d", item, interval, key_block, i, kb);
                        EXPECT(cut.first_interval(kb) <= i, "first_interval");
                        const int lo = std::max(i * length, visits.first_tile(kb)), hi = cut.end_of(i);
                        EXPECT(lo < hi, "empty item heads %d tokens %d length %d interval %d block %d", heads, tokens, length, i, kb);
                        for (int tile = lo; tile < hi; ++tile) ++seen[(size_t)kb * cut.row_tiles + tile];
                        ++parts[kb];
                    }
                }
                EXPECT(item == cut.items(), "items");
                for (int kb = 0; kb < cut.key_blocks; ++kb) {
                    EXPECT(parts[kb] == cut.intervals - cut.first_interval(kb), "parts of block %d: %d", kb, parts[kb]);
                    for (int tile = 0; tile < cut.row_tiles; ++tile) {
                        EXPECT(seen[(size_t)kb * cut.row_tiles + tile] == (tile >= visits.first_tile(kb) ? 1 : 0), "visit (%d, %d) seen %d times", kb, tile,
                               seen[(size_t)kb * cut.row_tiles + tile]);
                    }
                }
            }
        }
    }
}

// the interval length the dispatch picks by itself: known cases at 256 compute units (slots = rows * batch * 1024 bytes
// over 147456), and the bounds it promises wherever it picks one
void check_key_interval_choice() {
    struct { int tokens, heads, batch, expected; } known[] = {
        {4096, 128, 1, 192}, {2048, 128, 1, 96}, {1024, 128, 1, 48}, {512, 128, 1, 0}, {8192, 32, 1, 384},
        {2048, 16, 1, 0}, {4096, 128, 2, 384}, {16384, 16, 1, 768}, {1024, 128, 4, 48}, {300, 128, 8, 24}, {300, 128, 5, 24},
    };
    for (const auto& c : known) {
        const long long slots = (long long)c.tokens * c.heads * c.batch * 1024 / (2 * KEY_PARTIAL_BYTES);
        const int tiles = key_interval_choice(c.tokens, c.heads, c.batch, slots, 256, 2);
        EXPECT(tiles == c.expected, "interval choice T=%d H=%d B=%d: %d, expected %d", c.tokens, c.heads, c.batch, tiles, c.expected);
    }
    for (int heads : {1, 8, 16, 128}) {
        for (int tokens : {64, 1000, 4096, 20000}) {
            for (int batch : {1, 3}) {
                for (int units : {8, 256}) {
                    const long long slots = (long long)tokens * heads * batch * 1024 / (2 * KEY_PARTIAL_BYTES);
                    const int tiles = key_interval_choice(tokens, heads, batch, slots, units, 2);
                    if (tiles == 0) continue;
                    const long long items = key_intervals(tokens, heads, tiles, 2).items() * batch;
                    EXPECT(items <= slots && items <= 12LL * units && items >= 2LL * units, "items %lld of T=%d H=%d B=%d units %d", items,
                           tokens, heads, batch, units);
                }
            }
        }
    }
}

// ---- decode: the ranges partition the list of positions, their lengths differ by at most one, every tile of every
// sequence is computed by exactly one range, and (range, sequence) pairs that hold part of a sequence own distinct slots
void check_decode_ranges() {
    unsigned state = 12345;
    auto random = [&](int low, int high) { state = state * 1664525u + 1013904223u; return low + (int)((state >> 8) % (unsigned)(high - low + 1)); };
    for (int trial = 0; trial < 600; ++trial) {
        const int sequences = random(1, 70);
        int workgroups = random(1, 300);
        const int overhead = trial % 4 == 0 ? 0 : (trial % 4 == 1 ? SEGMENT_OVERHEAD : random(1, 9));
        std::vector<int> tiles(sequences), prefix(sequences + 1, 0);
        for (int s = 0; s < sequences; ++s) {
            tiles[s] = random(trial % 3 == 0 ? 0 : 1, trial % 2 ? 130 : 5);
            prefix[s + 1] = prefix[s] + positions_of(tiles[s], overhead);
        }
        const int total = prefix[sequences];
        if (total == 0) continue;
        const int launched = workgroups;
        workgroups = ranges_of(total, launched);   // the ranges the list is cut into
        EXPECT(workgroups >= 1 && workgroups <= launched && workgroups <= total, "%d ranges for %d positions, %d workgroups", workgroups, total, launched);
        std::set<int> slots;
        std::vector<std::vector<int>> covered(sequences);
        for (int s = 0; s < sequences; ++s) covered[s].assign(tiles[s], 0);
        EXPECT(range_begin_of(total, workgroups, 0) == 0 && range_begin_of(total, workgroups, workgroups) == total, "ends of the list");
        int shortest = total, longest = 0;
        for (int w = 0; w < workgroups; ++w) {
            const int begin = range_begin_of(total, workgroups, w), end = range_begin_of(total, workgroups, w + 1);
            EXPECT(end > begin, "workgroup %d range %d..%d", w, begin, end);
            shortest = std::min(shortest, end - begin);
            longest = std::max(longest, end - begin);
            for (int position = begin; position < end; ++position) {
                EXPECT(range_of_position(total, workgroups, position) == w, "position %d of %d, %d workgroups: owner %d, in range %d", position,
                       total, workgroups, range_of_position(total, workgroups, position), w);
            }
            for (int s = 0; s < sequences; ++s) {
                const int low = std::max(begin, prefix[s]), high = std::min(end, prefix[s + 1]);
                if (low >= high) continue;
                int first_tile, last_tile;
                tiles_in_positions(low, high, prefix[s], overhead, first_tile, last_tile);
                if (last_tile <= first_tile) continue;   // only positions of the sequence's overhead
                EXPECT(first_tile >= 0 && last_tile <= tiles[s], "sequence %d tiles %d..%d of %d", s, first_tile, last_tile, tiles[s]);
                for (int tile = first_tile; tile < last_tile; ++tile) ++covered[s][tile];
                const bool whole = first_tile == 0 && last_tile == tiles[s];
                int first, last;
                ranges_of_sequence(total, workgroups, prefix[s], prefix[s + 1] - prefix[s], overhead, first, last);
                EXPECT(first <= w && w <= last, "sequence %d is in range %d but its ranges are %d..%d", s, w, first, last);
                EXPECT(whole == (first == last), "sequence %d whole %d first %d last %d", s, (int)whole, first, last);
                if (!whole) {
                    const int slot = w + s;
                    EXPECT(slot < workgroups + sequences, "slot %d", slot);
                    EXPECT(slots.insert(slot).second, "slot %d used twice (workgroup %d sequence %d)", slot, w, s);
                }
            }
        }
        EXPECT(longest - shortest <= 1, "range lengths %d..%d", shortest, longest);
        for (int s = 0; s < sequences; ++s) {
            for (int tile = 0; tile < tiles[s]; ++tile) EXPECT(covered[s][tile] == 1, "sequence %d tile %d covered %d times", s, tile, covered[s][tile]);
            if (tiles[s] == 0) continue;
            // every range between the first and the last of a sequence holds some of its tiles (the merge reads them all)
            int first, last;
            ranges_of_sequence(total, workgroups, prefix[s], prefix[s + 1] - prefix[s], overhead, first, last);
            for (int w = first; w <= last; ++w) {
                const int begin = range_begin_of(total, workgroups, w), end = range_begin_of(total, workgroups, w + 1);
                int first_tile, last_tile;
                tiles_in_positions(std::max(begin, prefix[s]), std::min(end, prefix[s + 1]), prefix[s], overhead, first_tile, last_tile);
                EXPECT(last_tile > first_tile, "sequence %d: range %d of %d..%d holds none of its tiles", s, w, first, last);
            }
        }
    }
}

// ---- decode workspace: partial-result slots and the call's own plan stay inside the batch * heads * splits *
// (rank + 2) floats the caller provides, for every batch size, head count and split count; the plan's parts do not
// overlap
void check_decode_layout() {
    constexpr int RANK = 512, ROWS = 128;
    for (int compute_units : {1, 8, 256, 304}) {
        for (int batch = 1; batch <= 80; ++batch) {
            for (int heads : {1, 2, 16, 31, 32, 33, 127, 128, 129, 160, 256}) {
                for (int splits = 1; splits <= 34; ++splits) {
                    const DecodeLayout layout = decode_layout(batch, heads, splits, compute_units, ROWS, RANK);
                    const long long workspace = (long long)batch * heads * splits * (RANK + 2);
                    const int groups = (heads + ROWS - 1) / ROWS;
                    EXPECT(layout.head_groups == groups, "B %d H %d: %d head groups", batch, heads, layout.head_groups);
                    EXPECT(layout.workgroups >= 1 && layout.workgroups <= std::max(batch, compute_units), "B %d H %d splits %d: %d workgroups",
                           batch, heads, splits, layout.workgroups);
                    EXPECT(layout.plan_offset + layout.plan_ints <= workspace, "B %d H %d splits %d CUs %d: plan ends at %lld of %lld floats",
                           batch, heads, splits, compute_units, layout.plan_offset + layout.plan_ints, workspace);
                    EXPECT(layout.plan_ints == plan_elements(batch, layout.workgroups), "B %d H %d splits %d", batch, heads, splits);
                    // a slot holds 32 KB of bf16 accumulators per wave of 32 heads and two floats per head
                    const long long waves = (heads + 31) / 32;
                    EXPECT(layout.slot_floats * 4 == waves * 32768 + waves * 32 * 8, "H %d slot of %lld floats", heads, layout.slot_floats);
                    EXPECT(layout.slot_floats * 4 % 16 == 0, "H %d: slots must keep 16-byte alignment", heads);
                    if (layout.whole_sequences) {
                        EXPECT(layout.workgroups == batch && layout.slots == 0 && layout.plan_offset == 0, "B %d splits %d", batch, splits);
                    } else {
                        EXPECT(layout.workgroups >= 2 && layout.slots == layout.workgroups + batch, "B %d splits %d", batch, splits);
                        EXPECT(layout.plan_offset == layout.slots * layout.slot_floats, "B %d splits %d", batch, splits);
                        // as many workgroups as fit: one more would not
                        if (layout.workgroups < compute_units) {
                            const long long more = (layout.slots + 1) * layout.slot_floats + plan_elements(batch, layout.workgroups + 1);
                            EXPECT(more > workspace, "B %d H %d splits %d: %d workgroups but %d would fit", batch, heads, splits,
                                   layout.workgroups, layout.workgroups + 1);
                        }
                    }
                    // plan: header, prefix, first sequences follow one another
                    EXPECT(plan_prefix_at() == PLAN_HEADER && plan_first_sequence_at(batch) == PLAN_HEADER + batch + 1 &&
                               plan_elements(batch, layout.workgroups) == plan_first_sequence_at(batch) + layout.workgroups,
                           "plan parts B %d", batch);
                }
            }
        }
    }
    // the headline decode shape uses every compute unit
    const DecodeLayout headline = decode_layout(64, 128, 8, 256, ROWS, RANK);
    EXPECT(!headline.whole_sequences && headline.workgroups == 256, "B 64 H 128 splits 8: %d workgroups", headline.workgroups);
    // splits = 1 never cuts
    EXPECT(decode_layout(5, 128, 1, 256, ROWS, RANK).whole_sequences == 1, "splits 1 must not cut");
}

int main() {
    check_swizzle<128>();
    check_swizzle<256>();
    check_swizzle<384>();
    check_swizzle<1024>();
    check_swizzle<1152>();
    check_requests<384, 4>();
    check_requests<256, 4>();
    check_requests<128, 4>();
    check_requests<384, 8>();
    check_requests<256, 8>();
    check_requests<128, 8>();
    check_fragment_reads<128>();
    check_fragment_reads<256>();
    check_fragment_reads<384>();
    check_fragment_reads<1024>();
    check_fragment_reads<1152>();
    check_ds_blocks();
    check_forward_items();
    check_decode_loads<16>();
    check_decode_loads<8>();
    check_decode_loads<32>();
    check_key_visits();
    check_key_intervals();
    check_key_interval_choice();
    check_decode_ranges();
    check_decode_layout();
    if (failures) {
        std::printf("%d check(s) failed\n", failures);
        return 1;
    }
    std::printf("index_math: all checks passed\n");
    return 0;
}
