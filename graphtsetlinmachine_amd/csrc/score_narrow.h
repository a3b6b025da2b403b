// Clause evaluation on NARROW tiles, several clauses per wave.
//
// When a tile's rows are at most 64 words wide (graphs of 500 to 1,000 nodes whose thousand message
// rows have to share a workgroup's LDS: one or two graphs per tile), a wave that walks one clause's
// rows at a word per lane leaves lanes idle and reads LDS 256 bytes at a time, and a CU takes an
// LDS instruction only every four clocks or so whatever its width.  Here a GROUP of 8 or 16 lanes
// walks a clause of its own, WPL = 2 or 4 words per lane: lane l of a group holds words WPL l ..
// WPL l + WPL - 1 of the truth row of the group's clause.  Every row read (64 or 128 bits per
// lane), address add and AND serves 64 / GROUP clauses, and the waves of a workgroup are 64 or 128
// independent clause streams.  Shapes: (GROUP 16, WPL 2) for rows of at most 32 words, (16, 4) for
// rows of at most 64; (8, 4) - rows of at most 32 words on 128-bit reads - is kept for comparison.
//
// The same kernel evaluates
//   * a message layer (ROWS_MESSAGES; kernels.py:505-527): previous truth AND the rows of the
//     included message literals, complements for the negated ones - what k_tile_layer does, and
//   * layer 0 of a data set whose negated literals are the complements of its positive ones on
//     every node (ROWS_HALF; kernels.py:443-466 on what graphs.py:91-98,148-159 build; the caller
//     vouches for it with GTM_GRAPHS_COMPLEMENTARY): only the rows of the POSITIVE literals, the
//     node-type rows and the all-ones row are staged - half the rows, which is what lets a tile
//     of 2,048 literals into LDS at all - and a negated literal l + hv is the complement of row
//     l.  On node slots past a graph's nodes the complement is 1, but the node-type row, which
//     every clause ANDs first, is 0 there; the flag also says that no graph is empty.
//
// A clause's compiled list (k_compile_clauses with `half` set: header, rows to AND, rows whose
// complements to AND, each part a whole number of 8-entry blocks, filled up with the all-ones row
// to a whole number of 128 entries) is brought in by the group that evaluates it, a window of
// 4 GROUP entries at a time - one 16-byte load per lane, the first 96 or 128 entries requested two
// clauses ahead - and passes through a few words of LDS of the group's own, from which the walk
// reads it back a block ahead of the rows (the four lanes of a quad read entries 0..3 and 4..7 of
// a block, and an entry reaches all lanes inside the add that forms the row's address).  16 row
// words in flight per lane and trip (two blocks at 2 words per lane, one at 4), one test per two trips
// for "false at every node slot of the tile" - per group: a wave goes on while any of its clauses
// is alive and has rows left.  What differs between the groups in a trip - a block of rows to AND
// against a block of complements, a list that has ended - is a per-lane XOR mask folded into the
// AND (one three-input operation per pair of rows) and windows past a list's end replaced by the
// all-ones row.
//
// Between layers a stream also hands on WHICH of its clauses are still true somewhere in the tile
// (`alive`: per tile and stream a count and the clause numbers, written without atomics because a
// stream owns its clauses in every layer).  The next layer walks that list instead of testing the
// truth rows of all clauses - after the first message layer most are false everywhere.  The truth
// rows themselves stay complete: a clause that dies gets its row of zeros.
#pragma once
#include <type_traits>

constexpr int ROWS_HALF = 3;  // layer 0 on the positive literals' rows (+ node types, all ones), staged in LDS

constexpr int NARROW_WAVES = 16;
constexpr int NARROW_AHEAD = 2;         // clauses of a stream whose list and truth words are on their way
constexpr int NARROW_LIST_AHEAD = 128;  // entries of a clause's list requested with it (a list is at least as long)
constexpr int NARROW_MAX_STREAMS = 128;

// What depends on the lanes that share a clause.
template <int GROUP>
struct NarrowShape {
    static_assert(GROUP == 8 || GROUP == 16, "a half or a whole row of 16 lanes");
    static constexpr int PER_WAVE = 64 / GROUP;               // clauses under way in a wave
    static constexpr int STREAMS = PER_WAVE * NARROW_WAVES;   // clause streams of a workgroup
    static constexpr int WINDOW = 4 * GROUP;                  // list entries of a clause in LDS at a time: 4 per lane
    static constexpr int LIST_WORDS = WINDOW + 32;            // + what the walk reads ahead of the rows it is at
    // windows requested with the clause (of the 128 entries that every list has at least): 96 or 128 entries
    static constexpr int WINDOWS_AHEAD = NARROW_LIST_AHEAD / WINDOW > 3 ? 3 : NARROW_LIST_AHEAD / WINDOW;
};

struct NarrowArgs {
    const uint32_t *alive_in;  // [tiles of the launch][streams][alive_stride]: word 0 = n, then the stream's clauses
                               // that are true somewhere in the tile; NULL: every clause (q, q + streams, ...) is looked at
    uint32_t *alive_out;       // the same for the next layer, or NULL
    int alive_stride;          // >= 1 + ceil(C / streams)
    int alive_in_shared;       // alive_in is ONE set of lists for every tile (k_narrow_order_ranks: all clauses, by length)
    int hv, n_types;           // ROWS_HALF: positive literals (= LDS rows before the node-type rows), node types
    int row_words;             // words from one row to the next in LDS (>= tw, a multiple of 4): what the lists' entries count in
};

// The shape for a tile geometry: lanes per clause and words per lane (0, 0: none).  Rows of at most 32 words take
// 64-bit reads, four clauses per wave: with 128-bit reads a wave instruction covers eight rows at unrelated
// offsets, their bank conflicts cost more than the wider reads save (measured on 28-word rows: 5.7 against 4.7 ms),
// and 128 streams double the per-clause work around the walk.  `wide_reads` asks for that shape all the same
// (GTM_NARROW_READS=128, tuning and test aid).
struct NarrowChoice {
    int group, wpl;
    int streams() const { return group ? 64 / group * NARROW_WAVES : 0; }
    int list_words() const { return 4 * group + 32; }
};

inline NarrowChoice narrow_choice(const TileGeom &g, bool wide_reads = false) {
    // whole-word slots, rows a multiple of 4 words, built at one word per lane
    if (!g.ok || g.slot_words <= 0 || g.lw != 1 || g.tw % 4 != 0) return NarrowChoice{0, 0};
    if (g.tw <= 32) return wide_reads ? NarrowChoice{8, 4} : NarrowChoice{16, 2};
    if (g.tw <= 64) return NarrowChoice{16, 4};
    return NarrowChoice{0, 0};
}

inline int narrow_alive_stride(int C, int streams) { return 1 + (C + streams - 1) / streams; }

inline int narrow_rows_lds(int src, int M, int hv, int n_types) { return src == ROWS_HALF ? hv + n_types + 1 : M + 2; }

inline size_t narrow_lds_bytes(const TileGeom &g, const NarrowChoice &shape, int classes, int rows_lds, int row_words) {
    const size_t sums = ((size_t)g.gpt * classes + 3) & ~(size_t)3;  // the lists after them stay 16-byte aligned
    return ((size_t)rows_lds * row_words + TILE_LDS_PAD_WORDS + sums + (size_t)shape.streams() * shape.list_words()) * 4;
}

// Rows in LDS start 128 bytes apart where that fits: a group's read of a row then covers one aligned half of
// the 64 banks, and two groups of a wave collide only when their rows lie in the same half.  With rows 112 bytes
// apart (28-word rows as they lie in memory) nearly every pair of reads overlaps in some banks: a micro-benchmark
// of 16 waves reading four unrelated rows per 64-bit instruction takes 2.1 ns per instruction and CU at 112 bytes
// and 1.2 ns at 128.
inline int narrow_row_words(const TileGeom &g, const NarrowChoice &shape, int classes, int rows_lds, size_t lds_limit) {
    const int padded = (g.tw + 31) & ~31;
    return narrow_lds_bytes(g, shape, classes, rows_lds, padded) <= lds_limit ? padded : g.tw;
}

// The LDS addresses of a block's 8 rows for this lane: adr[i] = base + entry i of the block, where the
// four lanes of every quad hold entries 0..3 in `lo` and 4..7 in `hi`.  The entry comes across the quad
// inside the add (DPP); written out because the compiler folds such a lane move into the add only now
// and then.  (s_nop: a DPP operand written by the vector unit just before needs two idle states.)
__device__ __forceinline__ void narrow_block_addresses(uint32_t lo, uint32_t hi, uint32_t base, uint32_t (&adr)[8]) {
    asm volatile(
        "s_nop 1\n\t"
        "v_add_u32_dpp %0, %8, %10 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %1, %8, %10 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %2, %8, %10 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %3, %8, %10 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %4, %9, %10 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %5, %9, %10 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %6, %9, %10 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %7, %9, %10 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf bound_ctrl:1"
        : "=&v"(adr[0]), "=&v"(adr[1]), "=&v"(adr[2]), "=&v"(adr[3]), "=&v"(adr[4]), "=&v"(adr[5]), "=&v"(adr[6]),
          "=&v"(adr[7])
        : "v"(lo), "v"(hi), "v"(base));
}

// The same with the block's entries still in the registers they were fetched into: lane l of a group of 16 holds
// entries 4 l .. 4 l + 3 of the group's window of 64, so block BLOCK (entries 8 BLOCK ..) sits in lanes 2 BLOCK and
// 2 BLOCK + 1 of the group's row of 16 lanes, and an entry reaches all 16 lanes inside the add (row broadcast): the
// entries make no trip through LDS at all.
template <int BLOCK>
__device__ __forceinline__ void narrow_block_addresses_of_row(uint32_t e0, uint32_t e1, uint32_t e2, uint32_t e3,
                                                              uint32_t base, uint32_t (&adr)[8]) {
    asm volatile(
        "s_nop 1\n\t"
        "v_add_u32_dpp %0, %8, %12 row_newbcast:%13 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %1, %9, %12 row_newbcast:%13 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %2, %10, %12 row_newbcast:%13 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %3, %11, %12 row_newbcast:%13 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %4, %8, %12 row_newbcast:%14 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %5, %9, %12 row_newbcast:%14 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %6, %10, %12 row_newbcast:%14 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_add_u32_dpp %7, %11, %12 row_newbcast:%14 row_mask:0xf bank_mask:0xf bound_ctrl:1"
        : "=&v"(adr[0]), "=&v"(adr[1]), "=&v"(adr[2]), "=&v"(adr[3]), "=&v"(adr[4]), "=&v"(adr[5]), "=&v"(adr[6]),
          "=&v"(adr[7])
        : "v"(e0), "v"(e1), "v"(e2), "v"(e3), "v"(base), "n"(2 * BLOCK), "n"(2 * BLOCK + 1));
}

// AND of two rows that both come in as they are (flip = 0) or both inverted (flip = all ones): one
// three-input operation.
__device__ __forceinline__ uint32_t narrow_pair(uint32_t r0, uint32_t r1, uint32_t flip) {
    // truth table over (r0, r1, flip): 1 for (1, 1, 0) and for (0, 0, 1)
    return (uint32_t)__builtin_amdgcn_bitop3_b32((int)r0, (int)r1, (int)flip, 0x42);
}

__device__ __forceinline__ uint32_t narrow_and3(uint32_t a, uint32_t b, uint32_t c) {
    return (uint32_t)__builtin_amdgcn_bitop3_b32((int)a, (int)b, (int)c, 0x80);
}

typedef uint32_t narrow_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t narrow_u32x4 __attribute__((ext_vector_type(4)));
constexpr int NARROW_BUFFER_FLAGS = 0x00020000;  // last word of a buffer descriptor for plain 32-bit data on this GPU family

// The WPL words of a row that a lane holds (a native vector: the values stay in registers through copies and selects).
template <int WPL>
struct NarrowRow {
    typedef uint32_t Vec __attribute__((ext_vector_type(WPL)));
    Vec w;
    __device__ __forceinline__ bool any() const {
        uint32_t m = w[0];
#pragma unroll
        for (int u = 1; u < WPL; ++u) m |= w[u];
        return m != 0u;
    }
    __device__ __forceinline__ void fill(uint32_t v) { w = Vec(v); }
    __device__ __forceinline__ void load_lds(uint32_t address) {
        w = *(__attribute__((address_space(3))) const Vec *)(uintptr_t)address;
    }
    __device__ __forceinline__ void load(const uint32_t *p) { w = *reinterpret_cast<const Vec *>(p); }
    __device__ __forceinline__ void store(uint32_t *p) const { *reinterpret_cast<Vec *>(p) = w; }
    // through a buffer descriptor, at a 32-bit byte offset (no 64-bit address arithmetic per lane)
    __device__ __forceinline__ void load_at(__amdgpu_buffer_rsrc_t buffer, uint32_t at) {
        if (WPL == 2) {
            const narrow_u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(buffer, (int)at, 0, 0);
            w[0] = v.x, w[1] = v.y;
        } else {
            const narrow_u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(buffer, (int)at, 0, 0);
#pragma unroll
            for (int u = 0; u < WPL; ++u) w[u] = v[u];
        }
    }
    __device__ __forceinline__ void store_at(__amdgpu_buffer_rsrc_t buffer, uint32_t at) const {
        if (WPL == 2) {
            narrow_u32x2 v;
            v.x = w[0], v.y = w[1];
            __builtin_amdgcn_raw_buffer_store_b64(v, buffer, (int)at, 0, 0);
        } else {
            narrow_u32x4 v;
#pragma unroll
            for (int u = 0; u < WPL; ++u) v[u] = w[u];
            __builtin_amdgcn_raw_buffer_store_b128(v, buffer, (int)at, 0, 0);
        }
    }
};

typedef uint32_t NarrowEntries __attribute__((ext_vector_type(4)));  // four entries of a compiled list

// What the first lane of this lane's group of GROUP (16 or 8) lanes holds: a lane move inside the row of 16.
template <int GROUP>
__device__ __forceinline__ uint32_t narrow_group_first(uint32_t v, int lane) {
    const uint32_t of_row = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x150, 0xF, 0xF, true);  // row_share:0
    if (GROUP == 16) return of_row;
    const uint32_t of_upper = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x158, 0xF, 0xF, true);  // row_share:8
    return (lane & 8) ? of_upper : of_row;
}

// The greatest of a value that is the same in all lanes of a group, over the groups of the wave (wave-uniform):
// the rows of 16 lanes hand their value on to the next row and then to the upper half (row_bcast), lane 63 has it.
template <int GROUP>
__device__ __forceinline__ int narrow_max_over_groups(int v, int lane) {
    if (GROUP == 8) {
        const int other = __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true);  // row_ror:8: the row's other group
        v = v > other ? v : other;
    }
    const int from_row_before = __builtin_amdgcn_update_dpp(v, v, 0x142, 0xA, 0xF, false);  // row_bcast:15, rows 1 and 3
    v = v > from_row_before ? v : from_row_before;
    const int from_lower_half = __builtin_amdgcn_update_dpp(v, v, 0x143, 0xC, 0xF, false);  // row_bcast:31, rows 2 and 3
    v = v > from_lower_half ? v : from_lower_half;
    return __builtin_amdgcn_readlane(v, 63);
}

// Which clauses a stream takes when every clause is looked at (layer 0), in the format of the lists of clauses
// still alive: the clauses by falling length of their compiled lists, dealt out to the streams in turn - stream q
// takes ranks q, q + streams, ... - so that the groups of a wave, which stay together until the longest of their
// lists has been walked, hold lists of nearly the same length at every step, and a workgroup's long clauses come
// first.  The message layers take their clauses in the same order, as far as they are still alive, so among the
// clauses of one length in layer 0 (there are few different lengths) the order is by the length in the first
// message layer, then the second.  Ties by clause number: the table is the same from call to call.  Two launches:
// a key per clause (from entry 0 of each of its lists: blocks of rows | blocks of complements << 16), then a wave
// per clause that finds the clause's rank by counting the keys before its own, 64 at a time - work for the whole
// chip (a sort in one workgroup's LDS took 130 us for 8,000 clauses, this takes a fifth).
constexpr int NARROW_ORDER_BLOCK = 256;
constexpr int NARROW_ORDER_MAX_CLAUSES = 32768;
__global__ __launch_bounds__(NARROW_ORDER_BLOCK) void k_narrow_order_keys(const uint32_t *__restrict__ lists, int list_stride,
                                                                         const uint32_t *__restrict__ message_lists,
                                                                         int message_list_stride, int message_layers,
                                                                         int C, int streams, int alive_stride,
                                                                         uint32_t *__restrict__ keys, uint32_t *__restrict__ table) {
    const int c = blockIdx.x * NARROW_ORDER_BLOCK + threadIdx.x;
    // (a stream beyond the last clause has none; the launch has at least NARROW_ORDER_BLOCK >= streams threads)
    if (c < streams) table[(int64_t)c * alive_stride] = c < C ? (uint32_t)((C - c + streams - 1) / streams) : 0u;
    if (c >= C) return;
    auto blocks_of = [](uint32_t header) {
        const uint32_t n = (header & 0xFFFFu) + (header >> 16);
        return n < 1023u ? n : 1023u;
    };
    uint32_t h[3];
    h[0] = lists[(int64_t)c * list_stride];
#pragma unroll
    for (int l = 0; l < 2; ++l) h[1 + l] = l < message_layers ? message_lists[((int64_t)l * C + c) * message_list_stride] : 0u;
    keys[c] = blocks_of(h[0]) << 20 | blocks_of(h[1]) << 10 | blocks_of(h[2]);
}
static_assert(NARROW_ORDER_BLOCK >= NARROW_MAX_STREAMS, "one thread per stream writes its count");

__global__ __launch_bounds__(NARROW_ORDER_BLOCK) void k_narrow_order_ranks(const uint32_t *__restrict__ keys, int C, int streams,
                                                                          int alive_stride, uint32_t *__restrict__ table) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * (NARROW_ORDER_BLOCK / 64) + (threadIdx.x >> 6);
    if (c >= C) return;  // (whole waves)
    const uint32_t mine = keys[c];
    // clauses that come before this one: a greater key, or the same key and a smaller number
    int before = 0;
    for (int i0 = 0; i0 < C; i0 += 256) {
        uint32_t k[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + 64 * u + lane;
            k[u] = i < C ? keys[i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + 64 * u + lane;
            before += __popcll(__ballot(i < C && (k[u] > mine || (k[u] == mine && i < c))));
        }
    }
    if (lane == 0) table[(int64_t)(before % streams) * alive_stride + 1 + before / streams] = (uint32_t)c;
}

template <int SRC, bool LAST, int GROUP, int WPL>
__global__ __launch_bounds__(NARROW_WAVES * 64) void k_tile_layer_narrow(TileLayerArgs a, NarrowArgs x) {
    static_assert(SRC == ROWS_HALF || SRC == ROWS_MESSAGES, "layer 0 on half rows, or a message layer");
    static_assert(WPL == 2 || WPL == 4, "64- or 128-bit row reads");
    using Shape = NarrowShape<GROUP>;
    using Row = NarrowRow<WPL>;
    constexpr int PER = Shape::PER_WAVE, STREAMS = Shape::STREAMS, WINDOW = Shape::WINDOW, AHEAD_W = Shape::WINDOWS_AHEAD;
    constexpr int TRIP = 4 / WPL;  // blocks of 8 rows per trip: 16 row words in flight per lane
    constexpr uint32_t GROUP_MASK = (1u << GROUP) - 1u;
    extern __shared__ uint32_t lds[];
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, rw = x.row_words, C = a.C, K = a.K;
    constexpr int NT = NARROW_WAVES * 64;
    const int rows_lds = SRC == ROWS_HALF ? x.hv + x.n_types + 1 : a.M + 2;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)rows_lds * rw + TILE_LDS_PAD_WORDS);
    uint32_t *lists = (uint32_t *)sums + ((tg.gpt * K + 3) & ~3);
    const int tile_local = blockIdx.x, tile = a.tile0 + tile_local;
    const int tid = threadIdx.x, lane = tid & 63, gl = lane & (GROUP - 1), group = lane / GROUP;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = PER * wave + group;  // this group's stream
    uint32_t *bitmap = a.bitmap + (int64_t)tile_local * C * tw;
    // the compiled lists and this tile's truth rows, each through a buffer descriptor: an access is a multiply-add of
    // 24-bit factors per lane (clause x bytes per clause + the lane's place), not a 64-bit multiply and add
    const __amdgpu_buffer_rsrc_t lists_buffer =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(a.lists), 0, C * a.stride * 4, NARROW_BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t truth_buffer = __builtin_amdgcn_make_buffer_rsrc(bitmap, 0, C * tw * 4, NARROW_BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t weights_buffer =  // clause-major weights (last layer)
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t *>(LAST ? a.wt : nullptr), 0, LAST ? C * K * 4 : 0, NARROW_BUFFER_FLAGS);

    {  // rows -> LDS, 16 bytes per thread and trip, four loads in flight
        const uint4 *src;
        int first4, skip4;  // ROWS_HALF: the tile's rows hv .. 2 hv - 1 (the negated literals) stay out
        if (SRC == ROWS_HALF) {
            src = reinterpret_cast<const uint4 *>(a.tiles + (int64_t)tile * tg.rows * tw);
            first4 = (x.hv * tw) >> 2, skip4 = (x.hv * tw) >> 2;
        } else {
            src = reinterpret_cast<const uint4 *>(a.message_rows + (int64_t)tile_local * rows_lds * tw);
            first4 = 0x7FFFFFFF, skip4 = 0;
        }
        uint4 *dst = reinterpret_cast<uint4 *>(bt);
        const int n4 = (rows_lds * tw) >> 2;  // tw is a multiple of 4
        const int pieces = tw >> 2, apart = rw >> 2;  // 16-byte pieces of a row; from row to row in LDS
        for (int i = tid; i < n4; i += NT * 4) {
            uint4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int at = i + u * NT;
                v[u] = at < n4 ? src[at < first4 ? at : at + skip4] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int at = i + u * NT;
                if (at < n4) dst[rw == tw ? at : at / pieces * apart + at % pieces] = v[u];
            }
        }
        // the words after the rows read as zero (the complement of "no row": all ones), the class sums start at zero
        for (int i = tid; i < TILE_LDS_PAD_WORDS + ((tg.gpt * K + 3) & ~3); i += NT) bt[(size_t)rows_lds * rw + i] = 0;
    }
    __syncthreads();

    // Lanes past the row width keep a running AND of zero; they read the words after the row.
    const bool active = WPL * gl < tw;
    const uint32_t col_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t *)(bt + WPL * gl);
    uint32_t *my_list = lists + q * Shape::LIST_WORDS;
    const uint32_t *quad_entry = my_list + (lane & 3);
    const uint32_t ones_entry = (uint32_t)(rows_lds - 1 - (SRC == ROWS_MESSAGES ? 1 : 0)) * (uint32_t)rw * 4u;
    uint32_t ones_in_lane = ones_entry;  // (in a vector register: as a scalar operand of a select it costs a move each time)
    asm volatile("" : "+v"(ones_in_lane));
    // this group's lanes in a 64-bit vote: bits shift .. shift + GROUP - 1 of its low or high half
    const bool upper_half = lane >= 32;
    const uint32_t shift = (uint32_t)(group * GROUP) & 31u;
    auto votes_of_group = [&](unsigned long long vote) {
        const uint32_t half = upper_half ? (uint32_t)(vote >> 32) : (uint32_t)vote;
        return (half >> shift) & GROUP_MASK;
    };

    // slot bit 0 of the graphs without nodes (message layers): such a graph keeps every clause true
    Row empties;
    empties.fill(0u);
    bool any_empty = false;
    if (SRC == ROWS_MESSAGES) {
        if (active) empties.load(bt + (size_t)(a.M + 1) * rw + WPL * gl);
        any_empty = __ballot(empties.any()) != 0ull;
    }

    // this stream's clauses
    const uint32_t *seg_in =
        x.alive_in ? x.alive_in + ((int64_t)(x.alive_in_shared ? 0 : tile_local) * STREAMS + q) * x.alive_stride : nullptr;
    const int n_mine = seg_in ? (int)seg_in[0] : (q < C ? (C - q + STREAMS - 1) / STREAMS : 0);
    int n_most = 0;
#pragma unroll
    for (int g = 0; g < PER; ++g) n_most = max(n_most, __builtin_amdgcn_readlane(n_mine, g * GROUP));
    uint32_t *seg_out = x.alive_out ? x.alive_out + ((int64_t)tile_local * STREAMS + q) * x.alive_stride : nullptr;
    int n_out = 0;

    const int pairs = tg.gpt * K, sw = tg.slot_words;
    // Votes (last layer): lane p of a group adds weight k = p % K to graph j = p / K of the tile, for p = gl and
    // gl + GROUP; which class that is and which lanes of the group hold the graph's words (per word v of a lane:
    // ceil((w_lo - v) / WPL) <= l < ceil((w_hi - v) / WPL) for the graph's words [w_lo, w_hi)) does not depend on
    // the clause and is worked out once.  More (graph, class) pairs than that take the loop further down.
    constexpr int VOTES_AHEAD = 2;
    const bool votes_ahead = LAST && pairs <= VOTES_AHEAD * GROUP;
    int vote_class[VOTES_AHEAD];
    uint32_t vote_lanes[VOTES_AHEAD][WPL];
#pragma unroll
    for (int i = 0; i < VOTES_AHEAD; ++i) {
        const int p = gl + GROUP * i;
        const bool on = LAST && p < pairs;
        const int j = on ? p / K : 0;  // (a graph of the tile: the shifts below stay within the group's lanes)
        vote_class[i] = on ? p - j * K : 0;
        const int w_lo = j * sw, w_hi = w_lo + sw;
#pragma unroll
        for (int v = 0; v < WPL; ++v) {
            const int l_lo = (w_lo + WPL - 1 - v) / WPL, l_hi = (w_hi + WPL - 1 - v) / WPL;
            vote_lanes[i][v] = on ? ((1u << l_hi) - 1u) & ~((1u << l_lo) - 1u) : 0u;
        }
    }

    // The clause of item i of this stream (-1 past its end).  With a list of the clauses still alive, GROUP items
    // are held one per lane of the group and handed out with a lane read.
    uint32_t seg_now = 0u, seg_next = 0u;
    if (seg_in) {
        seg_now = gl < n_mine ? seg_in[1 + gl] : 0u;
        seg_next = GROUP + gl < n_mine ? seg_in[1 + GROUP + gl] : 0u;
    }
    auto clause_of = [&](int i) {
        if (i >= n_mine) return -1;
        if (!seg_in) return q + STREAMS * i;
        return (int)__shfl(seg_now, (lane & ~(GROUP - 1)) | (i & (GROUP - 1)));
    };
    struct Item {
        int c;              // the clause, -1: none
        NarrowEntries e[AHEAD_W];  // entries 4 gl .. 4 gl + 3 of the first windows of its list
        Row truth;          // its words of the clause's truth row (message layers)
    };
    auto fetch = [&](int i, Item &it) {  // item i's loads; i runs up by one from call to call
        if (seg_in && i > 0 && (i & (GROUP - 1)) == 0) {  // the next GROUP clauses of the stream's list move up
            seg_now = seg_next;
            seg_next = i + GROUP + gl < n_mine ? seg_in[1 + i + GROUP + gl] : 0u;
        }
        it.c = clause_of(i);
        const int c = it.c < 0 ? 0 : it.c;
        const uint32_t list_at = __umul24((uint32_t)c, (uint32_t)a.stride * 4u) + 16u * (uint32_t)gl;
#pragma unroll
        for (int v = 0; v < AHEAD_W; ++v)  // (a list is at least 128 entries long)
            it.e[v] = __builtin_amdgcn_raw_buffer_load_b128(lists_buffer, (int)list_at + v * WINDOW * 4, 0, 0);
        it.truth.fill(0u);
        if (SRC == ROWS_MESSAGES) it.truth.load_at(truth_buffer, __umul24((uint32_t)c, (uint32_t)tw * 4u) + (active ? 4u * WPL * gl : 0u));
    };

    // NARROW_AHEAD items are under way per stream: a clause's list and truth words come from L2 or further, a few
    // hundred cycles that one clause's evaluation does not cover.  The ring is unrolled so that each item keeps
    // registers of its own.
    Item ring[NARROW_AHEAD];
#pragma unroll
    for (int d = 0; d < NARROW_AHEAD; ++d) fetch(d, ring[d]);
    for (int i0 = 0; i0 < n_most; i0 += NARROW_AHEAD) {
#pragma unroll
        for (int d = 0; d < NARROW_AHEAD; ++d) {
            const Item now = ring[d];
            fetch(i0 + d + NARROW_AHEAD, ring[d]);
            if (i0 + d >= n_most) continue;  // (uniform over the wave)

            const bool has = now.c >= 0;
            const int c = has ? now.c : 0;
            Row truth_in, acc;
            truth_in.fill(0u);
            if (SRC == ROWS_MESSAGES && active && has) truth_in = now.truth;
            if (SRC == ROWS_MESSAGES)
                acc = truth_in;
            else
                acc.fill(active && has ? 0xFFFFFFFFu : 0u);
            // header (entry 0, in lane 0 of each group): blocks of rows to AND | blocks of rows whose complements to AND << 16
            const uint32_t header = narrow_group_first<GROUP>(now.e[0].x, lane);
            int plain = (int)(header & 0xFFFFu), nb = plain + (int)(header >> 16);
            unsigned long long nzw = __ballot(acc.any());
            const bool arrived_alive = votes_of_group(nzw) != 0u;
            if (!has || !arrived_alive) nb = 0, plain = 0;
            const int nb_most = narrow_max_over_groups<GROUP>(nb, lane);
            // does some group have a live clause with blocks left from block b on?
            auto work_left = [&](int b) { return __ballot(b < nb && votes_of_group(nzw) != 0u) != 0ull; };

            for (int b0 = 0; b0 < nb_most; b0 += WINDOW / 8) {  // one window of the lists after the other
                if (!work_left(b0)) break;
                NarrowEntries e;
                const int window = b0 / (WINDOW / 8);
                if (window < AHEAD_W) {
                    e = now.e[0];
#pragma unroll
                    for (int v = 1; v < AHEAD_W; ++v) e = window == v ? now.e[v] : e;
                } else {  // (a clause of more literals than that: its further windows are fetched when it gets there)
                    e = __builtin_amdgcn_raw_buffer_load_b128(
                        lists_buffer, (int)(__umul24((uint32_t)c, (uint32_t)a.stride * 4u) + 32u * (uint32_t)b0 + 16u * (uint32_t)gl), 0, 0);
                }
                // The compiled list is filled up with the all-ones row to a whole number of 128 entries.  A group
                // whose list has no such window (it ended in an earlier one; no clause; a clause false everywhere on
                // arrival: nb = 0) walks the all-ones row while the others go on.
                const bool past = b0 * 8 >= ((nb * 8 + NARROW_LIST_AHEAD - 1) & ~(NARROW_LIST_AHEAD - 1));
                if (past) e = NarrowEntries(ones_in_lane);
                if (b0 == 0 && gl == 0) e.x = ones_in_lane;  // in the place of the header
                const int lim_most = nb_most - b0 < WINDOW / 8 ? nb_most - b0 : WINDOW / 8;
                // bit b: block b0 + b of this group's list is one of complements (blocks plain .. nb - 1): its rows come in inverted
                const int from = plain - b0 < 0 ? 0 : plain - b0 > WINDOW / 8 ? WINDOW / 8 : plain - b0;
                const int to = nb - b0 < 0 ? 0 : nb - b0 > WINDOW / 8 ? WINDOW / 8 : nb - b0;
                const int flip_bits = to > from ? ((1 << to) - 1) & ~((1 << from) - 1) : 0;
                // TRIP blocks of 8 rows: read, and ANDed into the running truth
                auto and_rows = [&](const uint32_t (&adr)[TRIP][8], int at) {
                    Row r[TRIP][8];
#pragma unroll
                    for (int t = 0; t < TRIP; ++t)
#pragma unroll
                        for (int u = 0; u < 8; ++u) r[t][u].load_lds(adr[t][u]);
#pragma unroll
                    for (int t = 0; t < TRIP; ++t) {
                        // all ones for a block of complements, else zero (a signed one-bit field of flip_bits)
                        const uint32_t flip = (uint32_t)__builtin_amdgcn_sbfe(flip_bits, at + t, 1);
#pragma unroll
                        for (int v = 0; v < WPL; ++v) {
                            const uint32_t p0 = narrow_pair(r[t][0].w[v], r[t][1].w[v], flip);
                            const uint32_t p1 = narrow_pair(r[t][2].w[v], r[t][3].w[v], flip);
                            const uint32_t p2 = narrow_pair(r[t][4].w[v], r[t][5].w[v], flip);
                            const uint32_t p3 = narrow_pair(r[t][6].w[v], r[t][7].w[v], flip);
                            acc.w[v] = narrow_and3(narrow_and3(acc.w[v], p0, p1), p2, p3);
                        }
                    }
                };
                // Two trips between tests for "some group still has a live clause with blocks left": in the regime
                // that costs the time every clause walks its whole list, and the test is a sixth of a trip's vector
                // work.  (The blocks past a group's last one are the all-ones row: reading them changes nothing.)
                if constexpr (GROUP == 16) {
                    // the window's entries stay in the registers they came in (narrow_block_addresses_of_row): the walk
                    // over its 8 blocks is unrolled, every block's source lanes being fixed
                    bool go = true;
                    auto two_trips = [&](auto first_block) {
                        constexpr int b = decltype(first_block)::value;
                        if (!go) return;
                        if (!(b < lim_most && work_left(b0 + b))) {
                            go = false;
                            return;
                        }
                        auto trip = [&](auto first) {
                            constexpr int at = decltype(first)::value;
                            uint32_t adr[TRIP][8];
                            narrow_block_addresses_of_row<at>(e.x, e.y, e.z, e.w, col_lds, adr[0]);
                            if constexpr (TRIP == 2) narrow_block_addresses_of_row<at + 1>(e.x, e.y, e.z, e.w, col_lds, adr[TRIP - 1]);
                            and_rows(adr, at);
                        };
                        trip(std::integral_constant<int, b>{});
                        if (b + TRIP < lim_most) trip(std::integral_constant<int, b + TRIP>{});  // (else no group has a block there)
                        nzw = __ballot(acc.any());
                    };
                    two_trips(std::integral_constant<int, 0>{});
                    two_trips(std::integral_constant<int, 2 * TRIP>{});
                    if constexpr (TRIP == 1) {
                        two_trips(std::integral_constant<int, 4>{});
                        two_trips(std::integral_constant<int, 6>{});
                    }
                } else {
                    // groups of 8 lanes, two to a row of 16: the entries go through the group's words of LDS and come
                    // back a block ahead of the rows, four lanes of every quad on entries 0..3 and 4..7 of a block
                    *reinterpret_cast<NarrowEntries *>(my_list + 4 * gl) = e;
                    // (a wave's LDS accesses are carried out in order: the reads below see the entries just written)
                    uint32_t lo[TRIP], hi[TRIP];
#pragma unroll
                    for (int t = 0; t < TRIP; ++t) lo[t] = quad_entry[8 * t], hi[t] = quad_entry[8 * t + 4];
                    for (int b = 0; b < lim_most && work_left(b0 + b); b += 2 * TRIP) {
#pragma unroll
                        for (int half = 0; half < 2; ++half) {
                            const int at = b + half * TRIP;
                            if (half == 1 && at >= lim_most) break;  // (no group has a block there; uniform over the wave)
                            uint32_t n_lo[TRIP], n_hi[TRIP];
#pragma unroll
                            for (int t = 0; t < TRIP; ++t)
                                n_lo[t] = quad_entry[8 * (at + TRIP + t)], n_hi[t] = quad_entry[8 * (at + TRIP + t) + 4];
                            uint32_t adr[TRIP][8];
#pragma unroll
                            for (int t = 0; t < TRIP; ++t) narrow_block_addresses(lo[t], hi[t], col_lds, adr[t]);
                            and_rows(adr, at);
#pragma unroll
                            for (int t = 0; t < TRIP; ++t) lo[t] = n_lo[t], hi[t] = n_hi[t];
                        }
                        nzw = __ballot(acc.any());
                    }
                }
            }
            if (SRC == ROWS_MESSAGES && any_empty) {
#pragma unroll
                for (int v = 0; v < WPL; ++v) acc.w[v] = acc.w[v] | (truth_in.w[v] & empties.w[v]);
                nzw = __ballot(acc.any());
            }
            const uint32_t nzg = votes_of_group(nzw);  // this group's lanes with a true node slot
            if (has) {
                if (!LAST) {
                    // (a clause that was false everywhere on arrival has its row of zeros in place already)
                    if (active && (SRC == ROWS_HALF || arrived_alive))
                        acc.store_at(truth_buffer, __umul24((uint32_t)c, (uint32_t)tw * 4u) + 4u * WPL * gl);
                    if (seg_out && nzg != 0u) {
                        if (gl == 0) seg_out[1 + n_out] = (uint32_t)c;
                        ++n_out;
                    }
                } else if (nzg != 0u) {
                    // graph j of the tile owns words [j * sw, (j + 1) * sw) of the row; lane p of the group adds weight
                    // k = p % K to graph j = p / K, for p = gl, gl + GROUP, ...: which words of the group are non-zero
                    uint32_t nonzero[WPL];  // bit l: word WPL l + v
#pragma unroll
                    for (int v = 0; v < WPL; ++v) nonzero[v] = votes_of_group(__ballot(acc.w[v] != 0u));
                    const uint32_t weights_at = __umul24((uint32_t)c, (uint32_t)K * 4u);  // byte offset of the clause's weights
                    if (votes_ahead) {
#pragma unroll
                        for (int i = 0; i < VOTES_AHEAD; ++i) {
                            uint32_t hit = 0u;
#pragma unroll
                            for (int v = 0; v < WPL; ++v) hit |= nonzero[v] & vote_lanes[i][v];
                            if (hit)
                                atomicAdd(&sums[gl + GROUP * i],
                                          (int)__builtin_amdgcn_raw_buffer_load_b32(weights_buffer, (int)(weights_at + 4u * (uint32_t)vote_class[i]), 0, 0));
                        }
                    } else
                    for (int p = gl; p < pairs; p += GROUP) {
                        const int j = p / K, k = p - j * K;
                        const int w_lo = j * sw, w_hi = w_lo + sw;  // the graph's words
                        uint32_t hit = 0u;
#pragma unroll
                        for (int v = 0; v < WPL; ++v) {
                            // lanes whose word WPL l + v lies in [w_lo, w_hi): ceil((w_lo - v) / WPL) <= l < ceil((w_hi - v) / WPL)
                            const int l_lo = (w_lo + WPL - 1 - v) / WPL, l_hi = (w_hi + WPL - 1 - v) / WPL;
                            hit |= nonzero[v] & ((1u << l_hi) - 1u) & ~((1u << l_lo) - 1u);
                        }
                        if (hit)
                            atomicAdd(&sums[p], (int)__builtin_amdgcn_raw_buffer_load_b32(weights_buffer, (int)(weights_at + 4u * (uint32_t)k), 0, 0));
                    }
                }
            }
        }
    }
    if (!LAST) {
        if (seg_out && gl == 0) seg_out[0] = (uint32_t)n_out;
        return;
    }
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NT) {
        const int64_t g = g0 + i / K;
        if (g >= a.first_graph && g < (int64_t)a.first_graph + a.n_graphs)
            a.class_sum[(g - a.first_graph) * K + (i % K)] = sums[i];
    }
}
