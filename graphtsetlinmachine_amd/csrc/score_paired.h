// Clause evaluation on NARROW tiles, two clauses per wave.
//
// When a tile's rows are at most 32 words wide at one word per lane (graphs of 500 to 1,000 nodes
// whose thousand message rows have to share a workgroup's LDS: one graph per tile), a wave that
// walks one clause's rows has half its lanes idle.  Here each half of a wave walks a clause of its
// own: lane l and lane 32 + l hold word l of two different truth rows, every row read, address add
// and AND serves two clauses, and the waves of a workgroup are 32 independent clause streams.
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
// complements to AND, each part a whole number of 8-entry blocks) is brought in by the half-wave
// that evaluates it, 128 entries at a time - one 16-byte load per lane, requested one clause ahead
// - and passes through 160 words of LDS of the half-wave's own, from which the walk reads it back a
// block ahead of the rows (the four lanes of a quad read entries 0..3 and 4..7 of a block, and an
// entry reaches all lanes inside the add that forms the row's address).  Two blocks per trip, 16
// row reads in flight per lane, one test per trip for "false at every node slot of the tile" -
// per half: a wave goes on while either of its clauses is alive and has rows left.  What differs
// between the halves in a trip - a block of rows to AND against a block of complements, a list
// that has ended - is a per-lane XOR mask folded into the AND (one three-input operation) and
// list entries past the end replaced by the all-ones row.
//
// Between layers a stream also hands on WHICH of its clauses are still true somewhere in the tile
// (`alive`: per tile and stream a count and the clause numbers, written without atomics because a
// stream owns its clauses in every layer).  The next layer walks that list instead of testing the
// truth rows of all clauses - after the first message layer most are false everywhere.  The truth
// rows themselves stay complete: a clause that dies gets its row of zeros, because the kernels
// that build the messages read every clause's row.
#pragma once

constexpr int ROWS_HALF = 3;  // layer 0 on the positive literals' rows (+ node types, all ones), staged in LDS

constexpr int PAIRED_WAVES = 16;
constexpr int PAIRED_STREAMS = 2 * PAIRED_WAVES;
constexpr int PAIRED_WINDOW = 128;                     // list entries of a clause in LDS at a time: 4 per lane of a half-wave
constexpr int PAIRED_LIST_WORDS = PAIRED_WINDOW + 32;  // + what the walk reads ahead of the rows it is at
constexpr int PAIRED_AHEAD = 4;                        // clauses of a stream whose list and truth word are on their way

struct PairedArgs {
    const uint32_t *alive_in;  // [tiles of the launch][PAIRED_STREAMS][alive_stride]: word 0 = n, then the stream's clauses
                               // that are true somewhere in the tile; NULL: every clause (q, q + 32, ...) is looked at
    uint32_t *alive_out;       // the same for the next layer, or NULL
    int alive_stride;          // >= 1 + ceil(C / PAIRED_STREAMS)
    int hv, n_types;           // ROWS_HALF: positive literals (= LDS rows before the node-type rows), node types
};

inline int paired_alive_stride(int C) { return 1 + (C + PAIRED_STREAMS - 1) / PAIRED_STREAMS; }

inline int paired_rows_lds(int src, int M, int hv, int n_types) { return src == ROWS_HALF ? hv + n_types + 1 : M + 2; }

inline size_t paired_lds_bytes(const TileGeom &g, int classes, int rows_lds) {
    const size_t sums = ((size_t)g.gpt * classes + 3) & ~(size_t)3;  // the lists after them stay 16-byte aligned
    return ((size_t)rows_lds * g.tw + TILE_LDS_PAD_WORDS + sums + (size_t)PAIRED_STREAMS * PAIRED_LIST_WORDS) * 4;
}

// Geometry the kernel takes: whole-word slots, one word per lane, rows of at most 32 words.
inline bool paired_geometry(const TileGeom &g) { return g.ok && g.slot_words > 0 && g.lw == 1 && g.tw <= 32; }

typedef __attribute__((address_space(3))) const uint32_t *PairedLdsWord;

// The LDS addresses of a block's 8 rows for this lane: adr[i] = base + entry i of the block, where the
// four lanes of every quad hold entries 0..3 in `lo` and 4..7 in `hi`.  The entry comes across the quad
// inside the add (DPP); written out because the compiler folds such a lane move into the add only now
// and then.  (s_nop: a DPP operand written by the vector unit just before needs two idle states.)
__device__ __forceinline__ void paired_block_addresses(uint32_t lo, uint32_t hi, uint32_t base, uint32_t (&adr)[8]) {
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
__device__ __forceinline__ uint32_t paired_pair(uint32_t r0, uint32_t r1, uint32_t flip) {
    // truth table over (r0, r1, flip): 1 for (1, 1, 0) and for (0, 0, 1)
    return (uint32_t)__builtin_amdgcn_bitop3_b32((int)r0, (int)r1, (int)flip, 0x42);
}

template <int SRC, bool LAST>
__global__ __launch_bounds__(PAIRED_WAVES * 64) void k_tile_layer_paired(TileLayerArgs a, PairedArgs x) {
    static_assert(SRC == ROWS_HALF || SRC == ROWS_MESSAGES, "layer 0 on half rows, or a message layer");
    extern __shared__ uint32_t lds[];
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, C = a.C, K = a.K;
    constexpr int NT = PAIRED_WAVES * 64;
    const int rows_lds = SRC == ROWS_HALF ? x.hv + x.n_types + 1 : a.M + 2;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)rows_lds * tw + TILE_LDS_PAD_WORDS);
    uint32_t *lists = (uint32_t *)sums + ((tg.gpt * K + 3) & ~3);
    const int tile_local = blockIdx.x, tile = a.tile0 + tile_local;
    const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = 2 * wave + half;  // this half-wave's stream
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
    const bool active = l31 < tw;
    const uint32_t col_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t *)(bt + l31);
    uint32_t *my_list = lists + q * PAIRED_LIST_WORDS;
    const uint32_t *quad_entry = my_list + (lane & 3);
    const uint32_t ones_entry = (uint32_t)(rows_lds - 1 - (SRC == ROWS_MESSAGES ? 1 : 0)) * (uint32_t)tw * 4u;

    // slot bit 0 of the graphs without nodes (message layers): such a graph keeps every clause true
    uint32_t empties = 0u;
    bool any_empty = false;
    if (SRC == ROWS_MESSAGES) {
        empties = active ? bt[(size_t)(a.M + 1) * tw + l31] : 0u;
        any_empty = __ballot(empties != 0u) != 0ull;
    }

    // this stream's clauses
    const uint32_t *seg_in = x.alive_in ? x.alive_in + ((int64_t)tile_local * PAIRED_STREAMS + q) * x.alive_stride : nullptr;
    const int n_mine = seg_in ? (int)seg_in[0] : (q < C ? (C - q + PAIRED_STREAMS - 1) / PAIRED_STREAMS : 0);
    const int n_lo = __builtin_amdgcn_readlane(n_mine, 0), n_hi = __builtin_amdgcn_readlane(n_mine, 32);
    const int n_most = n_lo > n_hi ? n_lo : n_hi;
    uint32_t *seg_out = x.alive_out ? x.alive_out + ((int64_t)tile_local * PAIRED_STREAMS + q) * x.alive_stride : nullptr;
    int n_out = 0;

    // lane p of a half adds weight k = p % K to graph j = p / K of the tile, for p = l31, l31 + 32, ...
    const int pairs = tg.gpt * K, lpg = tg.lanes_per_graph;
    const uint32_t slot_lanes = lpg >= 32 ? 0xFFFFFFFFu : (1u << lpg) - 1u;

    // The clause of item i of this stream (-1 past its end).  With a list of the clauses still alive, 32 items
    // are held one per lane of the half-wave and handed out with a lane read.
    uint32_t seg_now = 0u, seg_next = 0u;
    if (seg_in) {
        seg_now = l31 < n_mine ? seg_in[1 + l31] : 0u;
        seg_next = 32 + l31 < n_mine ? seg_in[33 + l31] : 0u;
    }
    auto clause_of = [&](int i) {
        if (i >= n_mine) return -1;
        if (!seg_in) return q + PAIRED_STREAMS * i;
        return (int)__shfl(seg_now, (half << 5) | (i & 31));
    };
    struct Item {
        int c;          // the clause, -1: none
        uint4 e;        // entries 4 l31 .. 4 l31 + 3 of its list
        uint32_t truth; // word l31 of its truth row (message layers)
    };
    auto fetch = [&](int i, Item &it) {
        it.c = clause_of(i);
        const int c = it.c < 0 ? 0 : it.c;
        it.e = *reinterpret_cast<const uint4 *>(a.lists + (int64_t)c * a.stride + 4 * l31);
        it.truth = 0u;
        if (SRC == ROWS_MESSAGES) it.truth = bitmap[(int64_t)c * tw + (active ? l31 : 0)];
    };

    // PAIRED_AHEAD items are under way per stream: a clause's list and truth word come from L2 or further, a few
    // hundred cycles that one clause's evaluation does not cover.  The ring is unrolled so that each item keeps
    // registers of its own.
    auto fetch_next = [&](int i, Item &it) {  // item i's loads; i runs up by one from call to call
        if (seg_in && i > 0 && (i & 31) == 0) {  // the next 32 clauses of the stream's list move up
            seg_now = seg_next;
            seg_next = i + 32 + l31 < n_mine ? seg_in[i + 33 + l31] : 0u;
        }
        fetch(i, it);
    };
    Item ring[PAIRED_AHEAD];
#pragma unroll
    for (int d = 0; d < PAIRED_AHEAD; ++d) fetch_next(d, ring[d]);
    for (int i0 = 0; i0 < n_most; i0 += PAIRED_AHEAD) {
#pragma unroll
    for (int d = 0; d < PAIRED_AHEAD; ++d) {
        const Item now = ring[d];
        fetch_next(i0 + d + PAIRED_AHEAD, ring[d]);
        if (i0 + d >= n_most) continue;  // (uniform over the wave)

        const bool has = now.c >= 0;
        const int c = has ? now.c : 0;
        uint32_t truth_in = SRC == ROWS_MESSAGES && active && has ? now.truth : 0u;
        uint32_t acc = SRC == ROWS_MESSAGES ? truth_in : (active && has ? 0xFFFFFFFFu : 0u);
        // header (entry 0, in lane 0 of each half): blocks of rows to AND | blocks of rows whose complements to AND << 16
        const uint32_t header_lo = __builtin_amdgcn_readlane(now.e.x, 0), header_hi = __builtin_amdgcn_readlane(now.e.x, 32);
        const uint32_t header = half ? header_hi : header_lo;
        int plain = (int)(header & 0xFFFFu), nb = plain + (int)(header >> 16);
        unsigned long long nzw = __ballot(acc != 0u);
        bool alive_lo = (uint32_t)nzw != 0u, alive_hi = (uint32_t)(nzw >> 32) != 0u;
        const bool arrived_alive = half ? alive_hi : alive_lo;
        if (!has || !arrived_alive) nb = 0, plain = 0;
        const int nb_lo = __builtin_amdgcn_readlane(nb, 0), nb_hi = __builtin_amdgcn_readlane(nb, 32);
        const int nb_most = nb_lo > nb_hi ? nb_lo : nb_hi;

        uint4 e = now.e;
        for (int b0 = 0; b0 < nb_most; b0 += PAIRED_WINDOW / 8) {  // one window of the lists after the other
            if ((!alive_lo || b0 >= nb_lo) && (!alive_hi || b0 >= nb_hi)) break;
            if (b0 > 0) e = *reinterpret_cast<const uint4 *>(a.lists + (int64_t)c * a.stride + b0 * 8 + 4 * l31);
            // The compiled list is filled up with the all-ones row to the end of its last window.  A half-wave whose
            // list has no such window (it ended in an earlier one; no clause; a clause false everywhere on arrival:
            // nb = 0) walks the all-ones row while the other half goes on.
            const bool past = b0 * 8 >= ((nb * 8 + PAIRED_WINDOW - 1) & ~(PAIRED_WINDOW - 1));
            if (past) e = make_uint4(ones_entry, ones_entry, ones_entry, ones_entry);
            if (b0 == 0 && l31 == 0) e.x = ones_entry;  // in the place of the header
            *reinterpret_cast<uint4 *>(my_list + 4 * l31) = e;
            // (a wave's LDS accesses are carried out in order: the reads below see the entries just written)
            const int lim_lo = nb_lo - b0, lim_hi = nb_hi - b0;
            const int lim_most = nb_most - b0 < PAIRED_WINDOW / 8 ? nb_most - b0 : PAIRED_WINDOW / 8;
            uint32_t lo0 = quad_entry[0], hi0 = quad_entry[4], lo1 = quad_entry[8], hi1 = quad_entry[12];
            for (int b = 0; b < lim_most && ((alive_lo && b < lim_lo) || (alive_hi && b < lim_hi)); b += 2) {
                const uint32_t n_lo0 = quad_entry[8 * b + 16], n_hi0 = quad_entry[8 * b + 20];
                const uint32_t n_lo1 = quad_entry[8 * b + 24], n_hi1 = quad_entry[8 * b + 28];
                uint32_t adr0[8], adr1[8];
                paired_block_addresses(lo0, hi0, col_lds, adr0);
                paired_block_addresses(lo1, hi1, col_lds, adr1);
                uint32_t r[16];
#pragma unroll
                for (int u = 0; u < 8; ++u) r[u] = *(PairedLdsWord)(uintptr_t)adr0[u];
#pragma unroll
                for (int u = 0; u < 8; ++u) r[8 + u] = *(PairedLdsWord)(uintptr_t)adr1[u];
                // a block of complements for this half (blocks plain .. nb - 1 of its list): the rows come in inverted
                const int gb = b0 + b;
                uint32_t flip0 = gb >= plain && gb < nb ? 0xFFFFFFFFu : 0u;
                uint32_t flip1 = gb + 1 >= plain && gb + 1 < nb ? 0xFFFFFFFFu : 0u;
                asm("" : "+v"(flip0), "+v"(flip1));  // (plain words from here on: one three-input operation per pair of rows)
                uint32_t t[8];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    t[u] = paired_pair(r[2 * u], r[2 * u + 1], flip0);
                    t[4 + u] = paired_pair(r[8 + 2 * u], r[9 + 2 * u], flip1);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) acc &= t[u];
                nzw = __ballot(acc != 0u);
                alive_lo = (uint32_t)nzw != 0u, alive_hi = (uint32_t)(nzw >> 32) != 0u;
                lo0 = n_lo0, hi0 = n_hi0, lo1 = n_lo1, hi1 = n_hi1;
            }
        }
        if (SRC == ROWS_MESSAGES && any_empty) {
            acc |= truth_in & empties;
            nzw = __ballot(acc != 0u);
        }
        const uint32_t nzh = half ? (uint32_t)(nzw >> 32) : (uint32_t)nzw;  // this half's lanes with a true node slot
        if (has) {
            if (!LAST) {
                // (a clause that was false everywhere on arrival has its row of zeros in place already)
                if (active && (SRC == ROWS_HALF || arrived_alive)) bitmap[(int64_t)c * tw + l31] = acc;
                if (seg_out && nzh != 0u) {
                    if (l31 == 0) seg_out[1 + n_out] = (uint32_t)c;
                    ++n_out;
                }
            } else if (nzh != 0u) {
                const int32_t *weights_of_clause = a.wt + (int64_t)c * K;
                for (int p = l31; p < pairs; p += 32) {
                    const int j = p / K, k = p - j * K;
                    if ((nzh >> (j * lpg)) & slot_lanes) atomicAdd(&sums[p], weights_of_clause[k]);
                }
            }
        }
    }
    }
    if (!LAST) {
        if (seg_out && l31 == 0) seg_out[0] = (uint32_t)n_out;
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
