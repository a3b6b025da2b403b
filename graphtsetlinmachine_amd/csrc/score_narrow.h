// Clause evaluation on NARROW tiles, four clauses per wave.
//
// When a tile's rows are at most 32 words wide (graphs of 500 to 1,000 nodes whose thousand message
// rows have to share a workgroup's LDS: one graph per tile), a wave that walks one clause's rows at
// a word per lane has half its lanes idle - and reads LDS at half its rate, which 32-bit reads
// cannot exceed.  Here each QUARTER of a wave walks a clause of its own, two words per lane: lanes
// 16 g .. 16 g + 15 hold words 2 l, 2 l + 1 of the truth row of the clause of group g.  Every row
// read (64 bits per lane: the LDS at full rate), address add and AND serves four clauses, and the
// waves of a workgroup are 64 independent clause streams.
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
// to a whole number of windows) is brought in by the quarter-wave that evaluates it, a window of
// 64 entries at a time - one 16-byte load per lane, the first two windows requested two clauses ahead - and passes
// through 96 words of LDS of the quarter-wave's own, from which the walk reads it back a block
// ahead of the rows (the four lanes of a quad read entries 0..3 and 4..7 of a block, and an entry
// reaches all lanes inside the add that forms the row's address).  Two blocks per trip, 16 row
// reads in flight per lane, one test per trip for "false at every node slot of the tile" - per
// group: a wave goes on while any of its clauses is alive and has rows left.  What differs between
// the groups in a trip - a block of rows to AND against a block of complements, a list that has
// ended - is a per-lane XOR mask folded into the AND (one three-input operation per pair of rows)
// and windows past a list's end replaced by the all-ones row.
//
// Between layers a stream also hands on WHICH of its clauses are still true somewhere in the tile
// (`alive`: per tile and stream a count and the clause numbers, written without atomics because a
// stream owns its clauses in every layer).  The next layer walks that list instead of testing the
// truth rows of all clauses - after the first message layer most are false everywhere.  The truth
// rows themselves stay complete: a clause that dies gets its row of zeros, because the kernels
// that build the messages read every clause's row.
#pragma once

constexpr int ROWS_HALF = 3;  // layer 0 on the positive literals' rows (+ node types, all ones), staged in LDS

constexpr int NARROW_WAVES = 16;
constexpr int NARROW_GROUP = 16;                       // lanes that share a clause
constexpr int NARROW_PER_WAVE = 64 / NARROW_GROUP;     // clauses under way in a wave
constexpr int NARROW_STREAMS = NARROW_PER_WAVE * NARROW_WAVES;
constexpr int NARROW_WINDOW = 4 * NARROW_GROUP;        // list entries of a clause in LDS at a time: 4 per lane of its group
constexpr int NARROW_LIST_WORDS = NARROW_WINDOW + 32;  // + what the walk reads ahead of the rows it is at
constexpr int NARROW_AHEAD = 2;                        // clauses of a stream whose list and truth words are on their way
constexpr int NARROW_MAX_WORDS = 2 * NARROW_GROUP;     // widest row

struct NarrowArgs {
    const uint32_t *alive_in;  // [tiles of the launch][NARROW_STREAMS][alive_stride]: word 0 = n, then the stream's clauses
                               // that are true somewhere in the tile; NULL: every clause (q, q + 64, ...) is looked at
    uint32_t *alive_out;       // the same for the next layer, or NULL
    int alive_stride;          // >= 1 + ceil(C / NARROW_STREAMS)
    int hv, n_types;           // ROWS_HALF: positive literals (= LDS rows before the node-type rows), node types
};

inline int narrow_alive_stride(int C) { return 1 + (C + NARROW_STREAMS - 1) / NARROW_STREAMS; }

inline int narrow_rows_lds(int src, int M, int hv, int n_types) { return src == ROWS_HALF ? hv + n_types + 1 : M + 2; }

inline size_t narrow_lds_bytes(const TileGeom &g, int classes, int rows_lds) {
    const size_t sums = ((size_t)g.gpt * classes + 3) & ~(size_t)3;  // the lists after them stay 16-byte aligned
    return ((size_t)rows_lds * g.tw + TILE_LDS_PAD_WORDS + sums + (size_t)NARROW_STREAMS * NARROW_LIST_WORDS) * 4;
}

// Geometry the kernel takes: whole-word slots, rows of at most 32 words (a multiple of 4), built at one word per lane.
inline bool narrow_geometry(const TileGeom &g) { return g.ok && g.slot_words > 0 && g.lw == 1 && g.tw <= NARROW_MAX_WORDS; }

typedef uint32_t NarrowWords __attribute__((ext_vector_type(2)));  // the two words of a row that a lane holds
typedef __attribute__((address_space(3))) const NarrowWords *NarrowLdsWords;

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

// AND of two rows that both come in as they are (flip = 0) or both inverted (flip = all ones): one
// three-input operation.
__device__ __forceinline__ uint32_t narrow_pair(uint32_t r0, uint32_t r1, uint32_t flip) {
    // truth table over (r0, r1, flip): 1 for (1, 1, 0) and for (0, 0, 1)
    return (uint32_t)__builtin_amdgcn_bitop3_b32((int)r0, (int)r1, (int)flip, 0x42);
}

__device__ __forceinline__ uint32_t narrow_and3(uint32_t a, uint32_t b, uint32_t c) {
    return (uint32_t)__builtin_amdgcn_bitop3_b32((int)a, (int)b, (int)c, 0x80);
}

template <int SRC, bool LAST>
__global__ __launch_bounds__(NARROW_WAVES * 64) void k_tile_layer_narrow(TileLayerArgs a, NarrowArgs x) {
    static_assert(SRC == ROWS_HALF || SRC == ROWS_MESSAGES, "layer 0 on half rows, or a message layer");
    extern __shared__ uint32_t lds[];
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, C = a.C, K = a.K;
    constexpr int NT = NARROW_WAVES * 64;
    const int rows_lds = SRC == ROWS_HALF ? x.hv + x.n_types + 1 : a.M + 2;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)rows_lds * tw + TILE_LDS_PAD_WORDS);
    uint32_t *lists = (uint32_t *)sums + ((tg.gpt * K + 3) & ~3);
    const int tile_local = blockIdx.x, tile = a.tile0 + tile_local;
    const int tid = threadIdx.x, lane = tid & 63, gl = lane & (NARROW_GROUP - 1), group = lane / NARROW_GROUP;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = NARROW_PER_WAVE * wave + group;  // this group's stream
    uint32_t *bitmap = a.bitmap + (int64_t)tile_local * C * tw;

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
                if (at < n4) dst[at] = v[u];
            }
        }
        // the words after the rows read as zero (the complement of "no row": all ones), the class sums start at zero
        for (int i = tid; i < TILE_LDS_PAD_WORDS + ((tg.gpt * K + 3) & ~3); i += NT) bt[(size_t)rows_lds * tw + i] = 0;
    }
    __syncthreads();

    // Lanes past the row width keep a running AND of zero; they read the words after the row.
    const bool active = 2 * gl < tw;
    const uint32_t col_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t *)(bt + 2 * gl);
    uint32_t *my_list = lists + q * NARROW_LIST_WORDS;
    const uint32_t *quad_entry = my_list + (lane & 3);
    const uint32_t ones_entry = (uint32_t)(rows_lds - 1 - (SRC == ROWS_MESSAGES ? 1 : 0)) * (uint32_t)tw * 4u;
    const int shift16 = group * NARROW_GROUP;  // this group's lanes in a 64-bit vote

    // slot bit 0 of the graphs without nodes (message layers): such a graph keeps every clause true
    uint2 empties = make_uint2(0u, 0u);
    bool any_empty = false;
    if (SRC == ROWS_MESSAGES) {
        if (active) empties = *reinterpret_cast<const uint2 *>(bt + (size_t)(a.M + 1) * tw + 2 * gl);
        any_empty = __ballot((empties.x | empties.y) != 0u) != 0ull;
    }

    // this stream's clauses
    const uint32_t *seg_in = x.alive_in ? x.alive_in + ((int64_t)tile_local * NARROW_STREAMS + q) * x.alive_stride : nullptr;
    const int n_mine = seg_in ? (int)seg_in[0] : (q < C ? (C - q + NARROW_STREAMS - 1) / NARROW_STREAMS : 0);
    int n_most = 0;
#pragma unroll
    for (int g = 0; g < NARROW_PER_WAVE; ++g) n_most = max(n_most, __builtin_amdgcn_readlane(n_mine, g * NARROW_GROUP));
    uint32_t *seg_out = x.alive_out ? x.alive_out + ((int64_t)tile_local * NARROW_STREAMS + q) * x.alive_stride : nullptr;
    int n_out = 0;

    const int pairs = tg.gpt * K, sw = tg.slot_words;

    // The clause of item i of this stream (-1 past its end).  With a list of the clauses still alive, 16 items
    // are held one per lane of the group and handed out with a lane read.
    uint32_t seg_now = 0u, seg_next = 0u;
    if (seg_in) {
        seg_now = gl < n_mine ? seg_in[1 + gl] : 0u;
        seg_next = NARROW_GROUP + gl < n_mine ? seg_in[1 + NARROW_GROUP + gl] : 0u;
    }
    auto clause_of = [&](int i) {
        if (i >= n_mine) return -1;
        if (!seg_in) return q + NARROW_STREAMS * i;
        return (int)__shfl(seg_now, shift16 | (i & (NARROW_GROUP - 1)));
    };
    struct Item {
        int c;        // the clause, -1: none
        uint4 e, e2;  // entries 4 gl .. 4 gl + 3 of the first and of the second window of its list
        uint2 truth;  // words 2 gl, 2 gl + 1 of its truth row (message layers)
    };
    auto fetch = [&](int i, Item &it) {  // item i's loads; i runs up by one from call to call
        if (seg_in && i > 0 && (i & (NARROW_GROUP - 1)) == 0) {  // the next 16 clauses of the stream's list move up
            seg_now = seg_next;
            seg_next = i + NARROW_GROUP + gl < n_mine ? seg_in[1 + i + NARROW_GROUP + gl] : 0u;
        }
        it.c = clause_of(i);
        const int c = it.c < 0 ? 0 : it.c;
        const uint4 *list = reinterpret_cast<const uint4 *>(a.lists + (int64_t)c * a.stride + 4 * gl);
        it.e = list[0];
        it.e2 = list[NARROW_WINDOW / 4];  // (a list is at least two windows long, filled up with the all-ones row)
        it.truth = make_uint2(0u, 0u);
        if (SRC == ROWS_MESSAGES) it.truth = *reinterpret_cast<const uint2 *>(bitmap + (int64_t)c * tw + (active ? 2 * gl : 0));
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
            uint2 truth_in = make_uint2(0u, 0u);
            if (SRC == ROWS_MESSAGES && active && has) truth_in = now.truth;
            uint2 acc = SRC == ROWS_MESSAGES ? truth_in : (active && has ? make_uint2(0xFFFFFFFFu, 0xFFFFFFFFu) : make_uint2(0u, 0u));
            // header (entry 0, in lane 0 of each group): blocks of rows to AND | blocks of rows whose complements to AND << 16
            uint32_t header = 0u;
#pragma unroll
            for (int g = 0; g < NARROW_PER_WAVE; ++g) {
                const uint32_t h = __builtin_amdgcn_readlane(now.e.x, g * NARROW_GROUP);
                header = group == g ? h : header;
            }
            int plain = (int)(header & 0xFFFFu), nb = plain + (int)(header >> 16);
            unsigned long long nzw = __ballot((acc.x | acc.y) != 0u);
            const bool arrived_alive = ((nzw >> shift16) & 0xFFFFull) != 0ull;
            if (!has || !arrived_alive) nb = 0, plain = 0;
            int nb_of[NARROW_PER_WAVE], nb_most = 0;
#pragma unroll
            for (int g = 0; g < NARROW_PER_WAVE; ++g) {
                nb_of[g] = __builtin_amdgcn_readlane(nb, g * NARROW_GROUP);
                nb_most = max(nb_most, nb_of[g]);
            }
            // does some group have a live clause with blocks left from block b on?
            auto work_left = [&](int b) {
                bool left = false;
#pragma unroll
                for (int g = 0; g < NARROW_PER_WAVE; ++g) left |= b < nb_of[g] && ((nzw >> (g * NARROW_GROUP)) & 0xFFFFull) != 0ull;
                return left;
            };

            uint4 e = now.e;
            for (int b0 = 0; b0 < nb_most; b0 += NARROW_WINDOW / 8) {  // one window of the lists after the other
                if (!work_left(b0)) break;
                if (b0 == NARROW_WINDOW / 8)
                    e = now.e2;
                else if (b0 > 0)  // (a clause of more than 126 literals: its further windows are fetched when it gets there)
                    e = *reinterpret_cast<const uint4 *>(a.lists + (int64_t)c * a.stride + b0 * 8 + 4 * gl);
                // The compiled list is filled up with the all-ones row to the end of its last window.  A group whose
                // list has no such window (it ended in an earlier one; no clause; a clause false everywhere on arrival:
                // nb = 0) walks the all-ones row while the others go on.
                const bool past = b0 * 8 >= ((nb * 8 + NARROW_WINDOW - 1) & ~(NARROW_WINDOW - 1));
                if (past) e = make_uint4(ones_entry, ones_entry, ones_entry, ones_entry);
                if (b0 == 0 && gl == 0) e.x = ones_entry;  // in the place of the header
                *reinterpret_cast<uint4 *>(my_list + 4 * gl) = e;
                // (a wave's LDS accesses are carried out in order: the reads below see the entries just written)
                const int lim_most = nb_most - b0 < NARROW_WINDOW / 8 ? nb_most - b0 : NARROW_WINDOW / 8;
                // bit b: block b0 + b of this group's list is one of complements (blocks plain .. nb - 1): its rows come in inverted
                const int from = plain - b0 < 0 ? 0 : plain - b0 > 8 ? 8 : plain - b0, to = nb - b0 < 0 ? 0 : nb - b0 > 8 ? 8 : nb - b0;
                const int flip_bits = to > from ? ((1 << to) - 1) & ~((1 << from) - 1) : 0;
                uint32_t lo0 = quad_entry[0], hi0 = quad_entry[4], lo1 = quad_entry[8], hi1 = quad_entry[12];
#pragma unroll 2
                for (int b = 0; b < lim_most && work_left(b0 + b); b += 2) {
                    const uint32_t n_lo0 = quad_entry[8 * b + 16], n_hi0 = quad_entry[8 * b + 20];
                    const uint32_t n_lo1 = quad_entry[8 * b + 24], n_hi1 = quad_entry[8 * b + 28];
                    uint32_t adr0[8], adr1[8];
                    narrow_block_addresses(lo0, hi0, col_lds, adr0);
                    narrow_block_addresses(lo1, hi1, col_lds, adr1);
                    NarrowWords r[16];
#pragma unroll
                    for (int u = 0; u < 8; ++u) r[u] = *(NarrowLdsWords)(uintptr_t)adr0[u];
#pragma unroll
                    for (int u = 0; u < 8; ++u) r[8 + u] = *(NarrowLdsWords)(uintptr_t)adr1[u];
                    // all ones for a block of complements, else zero (a signed one-bit field of flip_bits)
                    const uint32_t flip0 = (uint32_t)__builtin_amdgcn_sbfe(flip_bits, b, 1);
                    const uint32_t flip1 = (uint32_t)__builtin_amdgcn_sbfe(flip_bits, b + 1, 1);
                    uint32_t tx[8], ty[8];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        tx[u] = narrow_pair(r[2 * u].x, r[2 * u + 1].x, flip0);
                        ty[u] = narrow_pair(r[2 * u].y, r[2 * u + 1].y, flip0);
                        tx[4 + u] = narrow_pair(r[8 + 2 * u].x, r[9 + 2 * u].x, flip1);
                        ty[4 + u] = narrow_pair(r[8 + 2 * u].y, r[9 + 2 * u].y, flip1);
                    }
#pragma unroll
                    for (int u = 0; u < 8; u += 2) {
                        acc.x = narrow_and3(acc.x, tx[u], tx[u + 1]);
                        acc.y = narrow_and3(acc.y, ty[u], ty[u + 1]);
                    }
                    nzw = __ballot((acc.x | acc.y) != 0u);
                    lo0 = n_lo0, hi0 = n_hi0, lo1 = n_lo1, hi1 = n_hi1;
                }
            }
            if (SRC == ROWS_MESSAGES && any_empty) {
                acc.x |= truth_in.x & empties.x, acc.y |= truth_in.y & empties.y;
                nzw = __ballot((acc.x | acc.y) != 0u);
            }
            const uint32_t nzg = (uint32_t)(nzw >> shift16) & 0xFFFFu;  // this group's lanes with a true node slot
            if (has) {
                if (!LAST) {
                    // (a clause that was false everywhere on arrival has its row of zeros in place already)
                    if (active && (SRC == ROWS_HALF || arrived_alive))
                        *reinterpret_cast<uint2 *>(bitmap + (int64_t)c * tw + 2 * gl) = acc;
                    if (seg_out && nzg != 0u) {
                        if (gl == 0) seg_out[1 + n_out] = (uint32_t)c;
                        ++n_out;
                    }
                } else if (nzg != 0u) {
                    // graph j of the tile owns words [j * sw, (j + 1) * sw) of the row; lane p of the group adds weight
                    // k = p % K to graph j = p / K, for p = gl, gl + 16, ...: which words of the group are non-zero
                    const uint32_t even = (uint32_t)(__ballot(acc.x != 0u) >> shift16) & 0xFFFFu;  // bit l: word 2 l
                    const uint32_t odd = (uint32_t)(__ballot(acc.y != 0u) >> shift16) & 0xFFFFu;   // bit l: word 2 l + 1
                    const int32_t *weights_of_clause = a.wt + (int64_t)c * K;
                    for (int p = gl; p < pairs; p += NARROW_GROUP) {
                        const int j = p / K, k = p - j * K;
                        const int w_lo = j * sw, w_hi = w_lo + sw;  // the graph's words
                        // lanes whose even word lies in [w_lo, w_hi): ceil(w_lo / 2) .. ceil(w_hi / 2) - 1; odd word: w_lo / 2 .. w_hi / 2 - 1
                        const uint32_t even_lanes = ((1u << ((w_hi + 1) >> 1)) - 1u) & ~((1u << ((w_lo + 1) >> 1)) - 1u);
                        const uint32_t odd_lanes = ((1u << (w_hi >> 1)) - 1u) & ~((1u << (w_lo >> 1)) - 1u);
                        if ((even & even_lanes) | (odd & odd_lanes)) atomicAdd(&sums[p], weights_of_clause[k]);
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
