// Batched inference on literal-major tiles.
//
// The dense form of clause evaluation tests every clause against every word
// of every node (CLAUSES x nodes x LA_CHUNKS word operations per graph) and is
// bound by integer VALU throughput, not by HBM.  A clause is an AND of few
// literals, so this path turns the data instead: for a tile of graphs it keeps
// one bit-row per LITERAL (bit n of the row = that literal at node slot n of
// the tile), staged in LDS, and a clause's truth over all node slots of the
// tile is the AND of the rows of its included literals only.  The result is
// the same bits as kernels.py:443-466 computes.  At depth 1 no clause/node
// bitmap is written because `evaluate` (kernels.py:297-315) only needs "true
// at some node of the graph"; with message layers the truth rows of a launch's
// tiles pass from layer to layer in the same slot layout, and each layer's
// messages are built literal-major as well.
//
// Tile layout in HBM (built once per data set by k_build_tiles):
//   tiles[tile][row][tw] uint32, rows = LITERALS + node_types + 1
//     row l < LITERALS          bit-row of literal l
//     row LITERALS + t          valid nodes of node type t
//     last row                  all ones (pads literal lists)
//   node slots: graph j of the tile owns `slot_bits` consecutive bits starting
//   at j * slot_bits; slot_bits is a power of two < 32 for tiny graphs, else a
//   whole number of 32-bit words (a multiple of the words one lane holds).
#pragma once

// Workgroup barrier for exchanges through LDS only: earlier LDS accesses of the wave are complete
// and visible to the group afterwards, but loads from (and atomics on) global memory stay in flight
// across it, which __syncthreads() would wait for.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct TileGeom {
    int slot_bits;        // bits per graph slot
    int slot_words;       // words per graph slot (0 when slot_bits < 32)
    int gpt;              // graphs per tile
    int tw;               // words per tile row
    int rows;             // LITERALS + node types + 1
    int n_tiles;
    int lw;               // words of a row held by one lane (1, 2 or 4)
    int lanes_per_graph;  // slot_words / lw (0 when slot_bits < 32)
    int ok;               // geometry supported by the tile kernels
    int stage0;           // the literal rows of layer 0 fit in LDS (else they are read from global memory)
    int half;             // layer 0 keeps only the rows of the positive literals in LDS and evaluates a negated
                          // literal as the complement of its positive row (k_tile_two_phase_half)
};

constexpr size_t TILE_LDS_BUDGET = 156 * 1024;  // of the 160 KB per CU
constexpr int TILE_LDS_PAD_WORDS = 256;         // readable words after the last row

inline size_t tile_lds_bytes(int rows, const TileGeom &g, int classes) {
    return ((size_t)rows * g.tw + TILE_LDS_PAD_WORDS + (size_t)g.gpt * classes) * 4;
}

// Tile shape for `lw` words per lane whose `fit_rows` rows fit in LDS (ok = 0 if none does).
inline TileGeom tile_geometry_lw(int literals, int n_types, int max_nodes, int n_graphs, int classes, int lw,
                                 int fit_rows) {
    TileGeom g{};
    g.lw = lw;
    g.rows = literals + n_types + 1;
    const int max_words = 64 * lw;
    if (max_nodes <= 16) {
        int s = 1;
        while (s < max_nodes) s <<= 1;
        g.slot_bits = s;
        // many rows: narrower rows (fewer graphs per tile) until the tile fits in LDS
        g.tw = max_words;
        g.gpt = g.tw * 32 / s;
        while (g.tw > 4 * lw && tile_lds_bytes(fit_rows, g, classes) > TILE_LDS_BUDGET) {
            g.tw >>= 1;
            g.gpt = g.tw * 32 / s;
        }
    } else {
        g.slot_words = ((max_nodes - 1) / 32 + 1 + lw - 1) / lw * lw;
        g.slot_bits = g.slot_words * 32;
        g.lanes_per_graph = g.slot_words / lw;
        g.gpt = g.slot_words <= max_words ? max_words / g.slot_words : 0;
        // fewer graphs per tile until the rows fit
        while (g.gpt > 1 && ((size_t)fit_rows * (((size_t)g.gpt * g.slot_words + 3) & ~(size_t)3) +
                             TILE_LDS_PAD_WORDS + (size_t)g.gpt * classes) * 4 > TILE_LDS_BUDGET)
            --g.gpt;
        g.tw = (g.gpt * g.slot_words + 3) & ~3;  // rows stay 16-byte aligned
        // nearly 64 lanes wide: widen the rows to all 64 lanes if that fits (the extra words are zero in
        // the node-type rows, so kernels need not mask the last lanes off)
        if (g.gpt > 0 && g.tw * 4 >= max_words * 3 && g.tw < max_words) {
            TileGeom wide = g;
            wide.tw = max_words;
            if (tile_lds_bytes(fit_rows, wide, classes) <= TILE_LDS_BUDGET) g.tw = max_words;
        }
    }
    g.n_tiles = g.gpt > 0 ? (n_graphs + g.gpt - 1) / g.gpt : 0;
    // (compiled clauses address a tile's rows by 31-bit byte offsets: bit 31 marks a negated message literal)
    g.ok = g.gpt > 0 && tile_lds_bytes(fit_rows, g, classes) <= TILE_LDS_BUDGET && (int64_t)g.rows * g.tw * 4 < (1ll << 31);
    g.stage0 = g.ok && tile_lds_bytes(g.rows, g, classes) <= TILE_LDS_BUDGET;
    return g;
}

// The lane width with the fewest wave instructions per graph whose tile fits in LDS: one step of
// a clause costs a wave one LDS read and `lw` ANDs whatever the number of lanes in use, and covers
// `gpt` graphs.  `message_rows` > 0 (models with message layers) asks that that many rows fit too;
// if the literal rows of layer 0 and the message rows cannot both fit, the message rows win and
// layer 0 reads its rows from global memory.
// Rows of layer 0 that a half tile keeps in LDS: the positive literals, the node types, all ones.
inline int tile_half_rows(int literals, int n_types) { return literals / 2 + n_types + 1; }

// `allow_half`: the data set's negated literals are the complements of its positive ones on every
// node and no graph is empty, so a tile may keep the positive rows only (TileGeom::half) - half the
// LDS per graph, which buys twice the graphs per tile.
inline TileGeom tile_geometry(int literals, int n_types, int max_nodes, int n_graphs, int classes, int max_lw = 4,
                              int message_rows = 0, bool allow_half = false, int half_lw = 0) {
    if (max_nodes < 1) max_nodes = 1;
    const int rows0 = literals + n_types + 1;
    if (allow_half && message_rows == 0 && max_nodes > 16) {
        TileGeom full = tile_geometry(literals, n_types, max_nodes, n_graphs, classes, max_lw, 0, false);
        TileGeom best_half{};
        for (int lw = max_lw; lw >= 1; lw >>= 1) {
            if (half_lw && lw != half_lw) continue;  // tuning aid: only this lane width, and then always taken
            TileGeom g = tile_geometry_lw(literals, n_types, max_nodes, n_graphs, classes, lw,
                                          tile_half_rows(literals, n_types));
            if (!g.ok) continue;
            if (!best_half.ok || (int64_t)(1 + g.lw) * best_half.gpt < (int64_t)(1 + best_half.lw) * g.gpt) best_half = g;
        }
        // taken when it covers more graphs per wave instruction than the tile of all rows
        if (best_half.ok && (!full.ok || !full.stage0 || half_lw ||
                             (int64_t)(1 + best_half.lw) * full.gpt < (int64_t)(1 + full.lw) * best_half.gpt)) {
            best_half.half = 1;
            best_half.stage0 = 1;
            return best_half;
        }
        return full;
    }
    TileGeom best{};
    for (int pass = 0; pass < 2; ++pass) {
        const int fit_rows = pass == 0 ? (rows0 > message_rows ? rows0 : message_rows) : message_rows;
        if (pass == 1 && message_rows == 0) break;
        for (int lw = max_lw; lw >= 1; lw >>= 1) {
            TileGeom g = tile_geometry_lw(literals, n_types, max_nodes, n_graphs, classes, lw, fit_rows);
            if (!g.ok) {
                if (!best.ok) best = g;
                continue;
            }
            // (1 + lw) / gpt, compared without division; ties go to the wider lanes
            if (!best.ok || (int64_t)(1 + g.lw) * best.gpt < (int64_t)(1 + best.lw) * g.gpt) best = g;
        }
        if (best.ok) {
            // Tiny graphs (several per word) whose many literal rows fit in LDS only at a fraction of the
            // 64 lanes' width: full-width rows read in place (global memory, L2) keep every lane busy
            // and leave few, large tiles, whose clauses several workgroups then share.
            if (message_rows == 0 && best.slot_words == 0 && best.tw < 64 * best.lw) {
                TileGeom wide = tile_geometry_lw(literals, n_types, max_nodes, n_graphs, classes, best.lw, 0);
                if (wide.ok && wide.tw > best.tw) return wide;
            }
            return best;
        }
    }
    best.ok = 0;
    return best;
}

// One thread per tile word: gathers its 32 node slots.
__global__ void k_build_tiles(const uint32_t *__restrict__ X, const uint32_t *__restrict__ node_type,
                              const uint32_t *__restrict__ node_index, const uint32_t *__restrict__ n_nodes_arr,
                              int G, int LA, int literals, int n_types, TileGeom tg, int64_t total,
                              uint32_t *__restrict__ tiles) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int w = (int)(i % tg.tw);
    int64_t rest = i / tg.tw;
    int row = (int)(rest % tg.rows);
    int tile = (int)(rest / tg.rows);
    uint32_t out = 0;
    if (row == tg.rows - 1) {
        // all ones over the graph slots; words that only pad the row stay 0 so
        // that they never keep a clause alive
        out = (tg.slot_words == 0 || w < tg.gpt * tg.slot_words) ? 0xFFFFFFFFu : 0u;
    } else {
        for (int b = 0; b < 32; ++b) {
            int pos = w * 32 + b;
            int j = pos / tg.slot_bits, n = pos % tg.slot_bits;
            int64_t g = (int64_t)tile * tg.gpt + j;
            if (j >= tg.gpt || g >= G) continue;
            int count = (int)n_nodes_arr[g];
            if (count == 0 && n == 0) {
                // kernels.py:289-295,443-466: for a graph without nodes the reference's
                // chunk arithmetic leaves every clause true; slot bit 0 carries that.
                out |= 1u << b;
                continue;
            }
            if (n >= count) continue;
            int64_t node = (int64_t)node_index[g] + n;
            uint32_t bit;
            if (row < literals)
                bit = (X[node * LA + (row >> 5)] >> (row & 31)) & 1u;
            else
                bit = (int)node_type[node] == row - literals;
            out |= bit << b;
        }
    }
    tiles[i] = out;
}

// Half tiles: the positive half of the literal words of the node in every slot (zeros where the slot
// holds no node).  One thread per slot.
__global__ void k_build_xpos(const uint32_t *__restrict__ X, const uint32_t *__restrict__ node_index,
                             const uint32_t *__restrict__ n_nodes_arr, int G, int LA, TileGeom tg, int64_t slots,
                             uint32_t *__restrict__ xpos) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots) return;
    const int per_tile = tg.tw * 32;
    const int64_t tile = i / per_tile;
    const int pos = (int)(i - tile * per_tile);
    const int j = pos / tg.slot_bits, n = pos - j * tg.slot_bits;
    const int64_t g = tile * tg.gpt + j;
    const int half = LA / 2;
    const bool has_node = j < tg.gpt && g < G && (uint32_t)n < n_nodes_arr[g];
    const uint32_t *row = has_node ? X + ((int64_t)node_index[g] + n) * LA : X;
    for (int w = 0; w < half; ++w) xpos[i * half + w] = has_node ? row[w] : 0u;
}

// Number of set bits of every row over all tiles (how often a literal holds in
// this data set); row_count[rows], zeroed by the caller.
__global__ void k_row_counts(const uint32_t *__restrict__ tiles, TileGeom tg, int64_t total_rows,
                             unsigned long long *__restrict__ row_count) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total_rows) return;
    int row = (int)(i % tg.rows);
    const uint32_t *p = tiles + i * tg.tw;
    unsigned long long n = 0;
    for (int w = 0; w < tg.tw; ++w) n += __popc(p[w]);
    if (n) atomicAdd(&row_count[row], n);
}

// Literal rows ordered by how often they hold in the data set, rarest first:
// order[r] = literal with rank r under the key (row_count, literal).  One
// thread per literal counts the keys below its own.
__global__ void k_row_order(const unsigned long long *__restrict__ row_count, int literals,
                            uint32_t *__restrict__ order) {
    int l = blockIdx.x * blockDim.x + threadIdx.x;
    if (l >= literals) return;
    unsigned long long mine = row_count[l];
    int rank = 0;
    for (int m = 0; m < literals; ++m) {
        unsigned long long other = row_count[m];
        rank += (other < mine) || (other == mine && m < l);
    }
    order[rank] = (uint32_t)l;
}

// Per call, one wave per clause: the rows the clause ANDs together, as 32-bit
// LDS byte offsets (row * tw * 4).  Entry 0 = the 8-entry blocks in use (see
// the end of the kernel); with n_types > 0 entry 1 = the row of the clause's
// node type (kernels.py:447); then the clause's included literals, in `order`
// when given: the ones that hold least often come first, so the running AND
// dies (and the walk stops) as early as it can; the order does not change the
// result.  With half > 0 (message banks) literal l >= half is the negation of
// literal l - half: those come in a second part, as the offsets of the rows
// whose complements are ANDed.  The list starts with a chunk of 32 entries;
// unused entries point at the all-ones row.  Also, when `weights` is given,
// the weights clause-major.

__global__ void k_compile_clauses(const uint32_t *__restrict__ bank, int C, int chunks, int B, uint32_t filter,
                                  int literals, int half, int n_types, int type_base_row, int ones_row, int tw,
                                  int stride, const uint32_t *__restrict__ order, uint32_t *__restrict__ lists, int K,
                                  const int32_t *__restrict__ weights, int32_t *__restrict__ wt,
                                  uint32_t *__restrict__ longest = nullptr) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (c >= C) return;
    const uint32_t row_bytes = (uint32_t)tw * 4u;
    const uint32_t ones = (uint32_t)ones_row * row_bytes;
    uint32_t *list = lists + (int64_t)c * stride;
    const uint32_t *inc = bank + (int64_t)c * chunks * B + (B - 1);
    int n = 1;
    if (n_types > 0) {
        if (lane == 0) list[1] = (uint32_t)(type_base_row + c % n_types) * row_bytes;
        n = 2;
    }
    // With negated literals as complements of rows (half > 0: message layers) the list comes in two parts, each a
    // whole number of 8-entry blocks: the rows to AND, then the rows whose complements to AND - a block is all of
    // one kind, so the evaluation needs no per-entry flag.  `plain`: entries of the first part.
    // (the number of entries of the first part is a count of include bits: no walk needed for it)
    int plain = 0;
    for (int w = lane; w < chunks; w += 64) {
        uint32_t word = inc[(int64_t)w * B];
        if (w == chunks - 1) word &= filter;
        if (half > 0) word = w < (half >> 5) ? word : w == (half >> 5) ? word & ((1u << (half & 31)) - 1u) : 0u;
        plain += __popc(word);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) plain += __shfl_xor(plain, off);
    plain += n;
    const int plain_padded = (plain + 7) & ~7;
    // With at most 64 include words lane w keeps word w, and a literal's bit comes by a lane read instead of a
    // load that depends on the load of `order`.
    const bool in_lanes = chunks <= 64;
    uint32_t word_of_lane = 0u;
    if (in_lanes && lane < chunks) {
        word_of_lane = inc[(int64_t)lane * B];
        if (lane == chunks - 1) word_of_lane &= filter;
    }
    int n_neg = 0;
    for (int r0 = 0; r0 < literals; r0 += 64) {
        int r = r0 + lane;
        uint32_t lit = r < literals ? (order ? order[r] : (uint32_t)r) : 0u;
        uint32_t w = lit >> 5;
        uint32_t word;
        if (in_lanes) {
            word = (uint32_t)__shfl((int)word_of_lane, (int)w);
        } else {
            word = inc[(int64_t)w * B];
            if ((int)w == chunks - 1) word &= filter;
        }
        const bool included = r < literals && ((word >> (lit & 31)) & 1u);
        const bool negated = included && half > 0 && (int)lit >= half;
        const unsigned long long below = (1ull << lane) - 1ull;
        const unsigned long long plain_mask = __ballot(included && !negated), neg_mask = __ballot(negated);
        if (included && !negated) list[n + __popcll(plain_mask & below)] = lit * row_bytes;
        if (negated) list[plain_padded + n_neg + __popcll(neg_mask & below)] = (lit - (uint32_t)half) * row_bytes;
        n += __popcll(plain_mask);
        n_neg += __popcll(neg_mask);
    }
    for (int i = n + lane; i < plain_padded; i += 64) list[i] = ones;
    // The last block of complements is filled up with the row after the all-ones row: in a message layer's rows
    // that is the row of the graphs without nodes, zero at every node slot of every other graph - and what its
    // complement takes from a graph without nodes the evaluation puts back (such a graph keeps every clause true).
    const int neg_padded = (n_neg + 7) & ~7;
    for (int i = n_neg + lane; i < neg_padded; i += 64) list[plain_padded + i] = ones + row_bytes;
    const int padded = plain_padded + neg_padded;
    // (to a whole number of 128-entry windows: k_tile_layer_paired takes a list a window at a time)
    const int fill_to = padded < 32 ? 128 : (padded + 127) & ~127;
    for (int i = padded + lane; i < fill_to; i += 64) list[i] = ones;
    // entry 0: blocks of rows to AND | blocks of rows whose complements to AND << 16
    if (lane == 0) list[0] = (uint32_t)(plain_padded >> 3) | ((uint32_t)(neg_padded >> 3) << 16);
    // entries of the longest list (cleared by the caller).  Thousands of atomics on one word are carried out one after
    // the other, about 10 ns each: a clause first looks whether the word already holds as much (it only ever grows,
    // so an old value can only cause an atomic that was not needed, never miss one).
    if (longest && lane == 0 && (uint32_t)padded > __hip_atomic_load(longest, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        atomicMax(longest, (uint32_t)padded);
    if (weights)
        for (int k = lane; k < K; k += 64) wt[(int64_t)c * K + k] = weights[(int64_t)k * C + c];
}

struct alignas(32) Block8 {
    uint32_t v[8];
};
struct alignas(64) Chunk16 {
    uint32_t v[16];
};
struct alignas(128) Chunk32 {
    uint32_t v[32];
};

// LW words of a tile row per lane, with the load width that goes with it.
template <int LW>
struct LaneWords;
template <>
struct LaneWords<1> {
    uint32_t w[1];
    __device__ __forceinline__ void load(const char *p) { w[0] = *reinterpret_cast<const uint32_t *>(p); }
    __device__ __forceinline__ void store(char *p) const { *reinterpret_cast<uint32_t *>(p) = w[0]; }
};
template <>
struct LaneWords<2> {
    uint32_t w[2];
    __device__ __forceinline__ void load(const char *p) {
        uint2 v = *reinterpret_cast<const uint2 *>(p);
        w[0] = v.x;
        w[1] = v.y;
    }
    __device__ __forceinline__ void store(char *p) const { *reinterpret_cast<uint2 *>(p) = make_uint2(w[0], w[1]); }
};
template <>
struct LaneWords<4> {
    uint32_t w[4];
    __device__ __forceinline__ void load(const char *p) {
        uint4 v = *reinterpret_cast<const uint4 *>(p);
        w[0] = v.x;
        w[1] = v.y;
        w[2] = v.z;
        w[3] = v.w;
    }
    __device__ __forceinline__ void store(char *p) const {
        *reinterpret_cast<uint4 *>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

// Where a layer's bit-rows come from.
constexpr int ROWS_STAGED = 0;   // the data set's tile (literal rows of layer 0), copied to LDS
constexpr int ROWS_GLOBAL = 1;   // the data set's tile, read in place (rows too big for LDS)
constexpr int ROWS_MESSAGES = 2; // message rows, built in LDS from the previous layer's bitmap

struct TileLayerArgs {
    const uint32_t *tiles;  // data set tiles (layer 0)
    TileGeom tg;
    int C, K;
    const uint32_t *lists;  // compiled clauses of this layer's bank
    int stride;
    const int32_t *wt;      // clause-major weights (last layer)
    int tile0, first_graph, n_graphs;
    int32_t *class_sum;     // [n_graphs][K] (last layer)
    uint32_t *bitmap;       // [tiles of the launch][C][tw]: clause truth per node slot, read and written in place
    int M, G;               // message size; graphs in the data set
    const uint32_t *node_index, *n_nodes;
    const uint32_t *X;      // [nodes][LA] node-major literal words (two-phase layer 0)
    const uint32_t *message_rows;  // [tiles of the launch][M + 2][tw] (message layers, built by k_tile_pack_messages)
    const uint32_t *xpos;   // [tiles][tw * 32 slots][LA / 2]: the positive literal words by node slot (half tiles)
    int walk_factor;        // k_tile_two_phase_wide: a clause's rows are all walked when more than this many slots per
                            // literal survive phase 1
    const struct TileSegment *segments;  // k_tile_two_phase_half: which clauses of which tile each workgroup takes, or NULL:
                            // workgroup b takes tile b whole
    int lists_in_lds;       // message layers: LDS holds TILE_LIST_LDS_WORDS more words per wave for the clause lists
    const uint32_t *longest_list;  // entries of the layer's longest list (message layers)
};

// A wave of k_tile_layer keeps the list of the clause it evaluates in LDS when it has at most this many entries
// (+ 32 words that the walk reads ahead).
constexpr int TILE_LIST_ENTRIES = 256;
constexpr int TILE_LIST_LDS_WORDS = TILE_LIST_ENTRIES + 32;

// Rows a message layer keeps in LDS: M message rows, the all-ones row, the row of graphs without nodes.
inline int tile_message_rows(int M) { return M + 2; }

inline size_t tile_layer_lds_bytes(const TileGeom &g, int classes, int src, int M) {
    return tile_lds_bytes(src == ROWS_STAGED ? g.rows : src == ROWS_MESSAGES ? tile_message_rows(M) : 0, g, classes);
}

// ---- the message rows of a layer, for all tiles of a launch ------------------
//
// A message factors: the bits a node sends are the OR of the hypervector bits
// of the clauses true at it; what a neighbour receives along an edge of type t
// is that bit vector rotated by t (kernels.py:581).  Node slots are addressed
// by their position in the tile, so padding slots simply stay empty.
//   k_tile_node_messages  sent[tile][slot][MW] from the truth rows [tile][C][tw]
//   k_tile_edge_messages  got[tile][dst slot] |= rotate(sent[tile][slot], type)
//   k_tile_pack_messages  rows[tile][M + 2][tw]: got turned literal-major, the
//                         all-ones row, the row of graphs without nodes
// (got is cleared before every layer's k_tile_edge_messages)
// MW = ceil(M / 32) words per vector.

constexpr int TILE_MESSAGES_BLOCK = 1024;

// The word of the lane whose index differs in bit J (1 .. 16): lane moves on the vector unit (within quads,
// within rows of 16 lanes, and the swap of neighbouring rows of 16), which do not queue behind the LDS
// traffic of the other waves the way a shuffle through the LDS crossbar does.  Every lane of the 32 that
// exchange must be active.
template <int J>
__device__ __forceinline__ uint32_t tile_lane_xor(uint32_t v, int lane) {
    static_assert(J == 1 || J == 2 || J == 4 || J == 8 || J == 16, "one bit of the lane index");
    if constexpr (J == 1) {
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1, 0, 3, 2]
    } else if constexpr (J == 2) {
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);  // quad_perm [2, 3, 0, 1]
    } else if constexpr (J == 4) {
        // lane ^ 7 (the 8 lanes mirrored), then lane ^ 3 (the quad reversed)
        const int mirrored = __builtin_amdgcn_mov_dpp((int)v, 0x141, 0xF, 0xF, true);  // row_half_mirror
        return (uint32_t)__builtin_amdgcn_mov_dpp(mirrored, 0x1B, 0xF, 0xF, true);     // quad_perm [3, 2, 1, 0]
    } else if constexpr (J == 8) {
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xF, 0xF, true);  // row_ror 8
    } else {
        // the odd rows of 16 lanes of the first copy and the even rows of the second change places
        const auto swapped = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        return (lane & 16) ? swapped[0] : swapped[1];
    }
}

// Transposes the 32 x 32 bit matrix whose row i is the word of lane i (of each half of the wave):
// afterwards bit i of lane b's word is what bit b of lane i's word was.  Five exchanges of
// half-blocks with the lane 16, 8, 4, 2, 1 away.
template <int J, uint32_t M>
__device__ __forceinline__ uint32_t tile_transpose_step(uint32_t v, int lane) {
    // M: the columns whose index has bit J clear.  A lane whose index has bit J clear keeps those columns and takes
    // the partner's, moved up by J, for the others: (v & M) | ((p & M) << J); a lane with bit J set the other way
    // round: (v & ~M) | ((p >> J) & M).  Both are (v & keep) | (rotate(p) & ~keep) with a rotation by J to the left
    // resp. right - what the rotation carries round lands on columns that `keep` covers - so the two kinds of lanes
    // run the same three instructions (lane exchange, rotate, bit select) on per-lane constants, no branch.
    const uint32_t p = tile_lane_xor<J>(v, lane);
    const bool upper = (lane & J) != 0;
    const uint32_t keep = upper ? ~M : M, left = upper ? 32u - J : (uint32_t)J;
    const uint32_t turned = __builtin_rotateleft32(p, left);
    return (v & keep) | (turned & ~keep);
}

__device__ __forceinline__ uint32_t tile_transpose32(uint32_t v, int lane) {
    v = tile_transpose_step<16, 0x0000FFFFu>(v, lane);
    v = tile_transpose_step<8, 0x00FF00FFu>(v, lane);
    v = tile_transpose_step<4, 0x0F0F0F0Fu>(v, lane);
    v = tile_transpose_step<2, 0x33333333u>(v, lane);
    return tile_transpose_step<1, 0x55555555u>(v, lane);
}


// What a node sends (kernels.py:565-588) is the OR of the hypervector bits of the clauses true at
// it.  Turned round: bit p of the vectors of 32 nodes is the OR of the truth words of the clauses
// whose hypervector holds p - plain ORs of whole words, however many clauses are true, instead of
// one atomic per (true clause, node, bit); 32 such words (bits 32 j .. 32 j + 31) transposed are
// word j of the 32 nodes' vectors.  k_message_bit_index lists the clauses of every bit.

constexpr int BIT_INDEX_BLOCK = 1024;

// One block.  start[p] .. start[p + 1] index `clauses` for message bit p; `cursor` is M words of scratch.
__global__ __launch_bounds__(BIT_INDEX_BLOCK) void k_message_bit_index(const uint32_t *__restrict__ hv, int C, int MB,
                                                                       int M, uint32_t *start, uint32_t *cursor,
                                                                       uint32_t *clauses) {
    __shared__ uint32_t chunk_sum[BIT_INDEX_BLOCK];
    const int tid = threadIdx.x;
    for (int p = tid; p <= M; p += BIT_INDEX_BLOCK) start[p] = 0u;
    for (int p = tid; p < M; p += BIT_INDEX_BLOCK) cursor[p] = 0u;
    __syncthreads();
    for (int i = tid; i < C * MB; i += BIT_INDEX_BLOCK) {
        const uint32_t h = hv[i];
        if (h < (uint32_t)M) atomicAdd(&start[h + 1], 1u);
    }
    __syncthreads();
    // running sums of start[1 .. M]: a run of `per` entries per thread, then the runs' totals
    const int per = (M + BIT_INDEX_BLOCK - 1) / BIT_INDEX_BLOCK;
    const int first = 1 + tid * per, last = first + per < M + 1 ? first + per : M + 1;
    uint32_t sum = 0u;
    for (int p = first; p < last; ++p) sum += start[p];
    chunk_sum[tid] = sum;
    __syncthreads();
    for (int off = 1; off < BIT_INDEX_BLOCK; off <<= 1) {
        const uint32_t v = tid >= off ? chunk_sum[tid - off] : 0u;
        __syncthreads();
        chunk_sum[tid] += v;
        __syncthreads();
    }
    uint32_t run = tid ? chunk_sum[tid - 1] : 0u;
    for (int p = first; p < last; ++p) {
        run += start[p];
        start[p] = run;
    }
    __syncthreads();
    // start[p + 1] now counts the entries of bits 0 .. p, so bit p's entries begin at start[p]
    for (int i = tid; i < C * MB; i += BIT_INDEX_BLOCK) {
        const uint32_t h = hv[i];
        if (h < (uint32_t)M) clauses[start[h] + atomicAdd(&cursor[h], 1u)] = (uint32_t)(i / MB);
    }
}

constexpr int MESSAGE_WORDS_AT_ONCE = 8;  // truth words a lane ORs per clause of its bit: independent loads in flight

// word[u] = OR over the clauses that hold message bit p of word u of their truth rows (`rows`:
// word 0 of clause 0's row, `tw` words per row), for u < n_words.
__device__ __forceinline__ void message_bit_words(const uint32_t *__restrict__ rows, int tw, int n_words,
                                                  const uint32_t *__restrict__ bit_start,
                                                  const uint32_t *__restrict__ bit_clauses, int p, int M,
                                                  uint32_t (&word)[MESSAGE_WORDS_AT_ONCE]) {
#pragma unroll
    for (int u = 0; u < MESSAGE_WORDS_AT_ONCE; ++u) word[u] = 0u;
    if (p >= M || n_words <= 0) return;
    const uint32_t from = bit_start[p], to = bit_start[p + 1];
    for (uint32_t i = from; i < to; ++i) {
        const uint32_t *row = rows + (int64_t)bit_clauses[i] * tw;
#pragma unroll
        for (int u = 0; u < MESSAGE_WORDS_AT_ONCE; ++u)
            if (u < n_words) word[u] |= row[u];
    }
}

// What the node slots of a tile send, vectors in global memory (graphs too big for the kernel
// below).  A wave takes 32 message bits (word j of every vector), lane = word of the tile's truth
// rows: for each bit the rows of the bit's clauses are ORed (whole rows, coalesced; the clause
// numbers come in by one load per bit and are handed round with readlane), the 32 resulting rows
// are transposed inside each lane, 32 x 32 bits, and the lane stores word j of its 32 slots.
// Every word of sent is written (no clearing
// needed).  Tiles of at most 32 words are taken `pack` = 64 / tw at a time, lane l on word l % tw of tile
// l / tw of the group (the clause numbers of a bit are the same for every tile).
constexpr int NODE_MESSAGES_BY_BIT_WAVES = 4;

__global__ __launch_bounds__(64 * NODE_MESSAGES_BY_BIT_WAVES) void k_tile_node_messages_by_bit(
    const uint32_t *__restrict__ bitmap, int C, int tw, const uint32_t *__restrict__ bit_start,
    const uint32_t *__restrict__ bit_clauses, int M, int MW, int n_tiles, int pack, int blocks_per_group, int n_groups,
    uint32_t *__restrict__ sent) {
    __shared__ uint32_t stage_of_wave[NODE_MESSAGES_BY_BIT_WAVES][32][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Workgroups go to the 8 XCDs in turn, and each XCD has its own L2: the workgroups of a group of tiles - they read
    // the same truth rows, each for its own message bits - are given to one XCD, so that the rows come from memory
    // once and not once per XCD.  1-D grid of ceil(groups / 8) * 8 * blocks_per_group workgroups.
    const int xcd = blockIdx.x & 7, turn = blockIdx.x >> 3;
    const int block_of_group = turn % blocks_per_group, group = (turn / blocks_per_group) * 8 + xcd;
    if (group >= n_groups) return;
    const int j = block_of_group * NODE_MESSAGES_BY_BIT_WAVES + wave;
    if (j >= MW) return;  // the block has no barrier
    uint32_t(*stage)[64] = stage_of_wave[wave];
    const int sub = pack > 1 ? lane / tw : 0, word_of_lane = pack > 1 ? lane - sub * tw : lane;
    const int tile = group * pack + sub;
    const bool tile_exists = sub < pack && tile < n_tiles;
    const uint32_t *rows = bitmap + (int64_t)(tile_exists ? tile : group * pack) * C * tw;
    // lane i <= 32 holds where the clauses of bit 32 j + i begin (bits past M: nothing)
    const int p_of_lane = 32 * j + lane < M ? 32 * j + lane : M;
    const uint32_t start_of_lane = lane <= 32 ? bit_start[p_of_lane] : 0u;
    for (int w0 = 0; w0 < (pack > 1 ? 1 : tw); w0 += 64) {
        const int w = pack > 1 ? word_of_lane : w0 + lane;
        const bool active = tile_exists && w < tw;
        const uint32_t *col = rows + (active ? w : 0);
#pragma unroll 1
        for (int i = 0; i < 32; ++i) {
            const uint32_t from = __builtin_amdgcn_readlane(start_of_lane, i);
            const uint32_t to = __builtin_amdgcn_readlane(start_of_lane, i + 1);
            uint32_t acc = 0u;
            for (uint32_t k0 = from; k0 < to; k0 += 64u) {
                const uint32_t n = to - k0 < 64u ? to - k0 : 64u;
                const uint32_t clause_of_lane = (uint32_t)lane < n ? bit_clauses[k0 + lane] : 0u;
                for (uint32_t e = 0; e < n; e += 8u) {
                    uint32_t v[8];
#pragma unroll
                    for (uint32_t u = 0; u < 8u; ++u) {
                        const uint32_t c = __builtin_amdgcn_readlane(clause_of_lane, (e + u) & 63u);
                        v[u] = e + u < n ? col[(int64_t)c * tw] : 0u;
                    }
#pragma unroll
                    for (uint32_t u = 0; u < 8u; ++u) acc |= v[u];
                }
            }
            stage[i][lane] = active ? acc : 0u;
        }
        // (a wave's LDS writes are visible to its own later reads: same wave, in order)
        uint32_t a[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) a[i] = stage[i][lane];
        // a[i] bit b -> a[b] bit i: blocks of s x s bits swap across the diagonal, s = 16 .. 1
#pragma unroll
        for (int s = 16; s >= 1; s >>= 1) {
            const uint32_t m = s == 16 ? 0x0000FFFFu : s == 8 ? 0x00FF00FFu : s == 4 ? 0x0F0F0F0Fu : s == 2 ? 0x33333333u : 0x55555555u;
#pragma unroll
            for (int i = 0; i < 32; ++i)
                if ((i & s) == 0) {
                    const uint32_t t = ((a[i] >> s) ^ a[i + s]) & m;
                    a[i + s] ^= t;
                    a[i] ^= t << s;
                }
        }
        if (active) {
            uint32_t *out = sent + ((int64_t)tile * tw + w) * 32 * MW + j;
#pragma unroll
            for (int b = 0; b < 32; ++b) out[(int64_t)b * MW] = a[b];
        }
    }
}

// grid (ceil(tw / group), tiles); `group` consecutive words of every truth row of the tile per
// block (a power of two <= 16: one cache line per clause), dynamic LDS 32 * group * (MW | 1) words.
// Every word of sent is written (no clearing needed).
__global__ __launch_bounds__(TILE_MESSAGES_BLOCK) void k_tile_node_messages(
    const uint32_t *__restrict__ bitmap, int C, int tw, int group, const uint32_t *__restrict__ hv, int MB, int MW,
    uint32_t *__restrict__ sent) {
    // [32 * group slots][MW | 1], slot s at s * (MW | 1) + s / 32: lanes on neighbouring slots hit different
    // banks, and so do lanes on the same bit of different words of a row (32 slots apart)
    extern __shared__ uint32_t vec[];
    const int tid = threadIdx.x;
    const int w0 = blockIdx.x * group, tile = blockIdx.y;
    const int MWP = MW | 1;
    const int n_vec = 32 * group * MWP + group;
    for (int i = tid; i < n_vec; i += TILE_MESSAGES_BLOCK) vec[i] = 0u;
    __syncthreads();
    const int wl = tid & (group - 1), w = w0 + wl;
    const uint32_t *rows = bitmap + (int64_t)tile * C * tw;
    constexpr int AHEAD = 4;  // truth words in flight per thread
    const int step = TILE_MESSAGES_BLOCK / group;
    if (w < tw)
        for (int c0 = tid / group; c0 < C; c0 += AHEAD * step) {
            uint32_t words[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const int c = c0 + u * step;
                words[u] = c < C ? rows[(int64_t)c * tw + w] : 0u;
            }
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                uint32_t word = words[u];
                if (!word) continue;
                const int c = c0 + u * step;
                for (int j = 0; j < MB; ++j) {
                    const uint32_t h = hv[(int64_t)c * MB + j];
                    const uint32_t bit = 1u << (h & 31);
                    uint32_t *column = vec + (wl * 32) * MWP + wl + (h >> 5);
                    for (uint32_t m = word; m; m &= m - 1) atomicOr(&column[(__ffs(m) - 1) * MWP], bit);
                }
            }
        }
    __syncthreads();
    uint32_t *out = sent + ((int64_t)tile * tw + w0) * 32 * MW;
    const int n_out = (min(tw, w0 + group) - w0) * 32 * MW;
    for (int i = tid; i < n_out; i += TILE_MESSAGES_BLOCK) out[i] = vec[(i / MW) * MWP + ((i / MW) >> 5) + i % MW];
}

// One thread per (tile of the launch, node slot, vector word).
__global__ void k_tile_edge_messages(const uint32_t *__restrict__ sent, TileGeom tg, int tile0, int G, int M, int MW,
                                     const uint32_t *__restrict__ node_index, const uint32_t *__restrict__ n_nodes,
                                     const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
                                     const uint32_t *__restrict__ edge, int64_t total, uint32_t *got) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int j = (int)(i % MW);
    const int64_t slot_id = i / MW;  // tile of the launch * slots per tile + slot
    const int slots = tg.tw * 32;
    const int tile_local = (int)(slot_id / slots), pos = (int)(slot_id % slots);
    const int gj = pos / tg.slot_bits, n = pos - gj * tg.slot_bits;
    const int64_t g = (int64_t)(tile0 + tile_local) * tg.gpt + gj;
    if (gj >= tg.gpt || g >= G || (uint32_t)n >= n_nodes[g]) return;
    const uint32_t *v = sent + slot_id * MW;
    const int64_t row = (int64_t)node_index[g] + n;
    const uint32_t ne = n_edges[row];
    const int64_t e0 = edge_index[row];
    for (uint32_t e = 0; e < ne; ++e) {
        const uint32_t dst = edge[(e0 + e) * 2], shift = edge[(e0 + e) * 2 + 1] % (uint32_t)M;
        uint32_t word = 0;
        if ((M & 31) == 0) {
            // bit p of the result is bit (p - shift) mod M of v
            const int q = (int)(shift >> 5), r = (int)(shift & 31u);
            const int a = (j - q + MW) % MW, below = (a - 1 + MW) % MW;
            word = r ? (v[a] << r) | (v[below] >> (32 - r)) : v[a];
        } else {
            for (int b = 0; b < 32; ++b) {
                const int p = j * 32 + b;
                if (p >= M) break;
                const int from = (p + M - (int)shift) % M;
                word |= ((v[from >> 5] >> (from & 31)) & 1u) << b;
            }
        }
        if (word) atomicOr(&got[((int64_t)tile_local * slots + gj * tg.slot_bits + dst) * MW + j], word);
    }
}

// grid (ceil(tw / 2), tiles), 256 threads: the received vectors of 64 node slots go through LDS
// (read row by row, coalesced) and come out literal-major: wave v turns vector words v, v + 4, ...
// into rows 32 j .. 32 j + 31 (lane = slot, a 32 x 32 bit transposition across the lanes of each half).  Wave 0 also writes the all-ones
// row M and row M + 1 (slot bit 0 of the graphs without nodes: the reference's chunk arithmetic
// leaves every clause true for such a graph at every layer, kernels.py:443-466,505-527, which the
// message literals must not undo).  Dynamic LDS 64 * (MW + 1) words.
__global__ __launch_bounds__(256) void k_tile_pack_messages(const uint32_t *__restrict__ got, TileGeom tg, int tile0,
                                                             int G, int M, int MW,
                                                             const uint32_t *__restrict__ n_nodes,
                                                             uint32_t *__restrict__ rows, int blocks_per_tile, int n_tiles) {
    extern __shared__ uint32_t block[];  // [64 slots][MW + 1]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // (the workgroups of a tile write neighbouring words of the same rows: they are given to one XCD - workgroups go to
    // the 8 XCDs in turn - so that the words meet in one L2 before they go to memory.  1-D grid of
    // ceil(tiles / 8) * 8 * blocks_per_tile workgroups.)
    const int xcd = blockIdx.x & 7, turn = blockIdx.x >> 3;
    const int nb = turn % blocks_per_tile, tile_local = (turn / blocks_per_tile) * 8 + xcd;
    if (tile_local >= n_tiles) return;
    const int tw = tg.tw, slots = tw * 32;
    const int n_here = min(64, slots - nb * 64);
    const uint32_t *src = got + ((int64_t)tile_local * slots + nb * 64) * MW;
    for (int i = tid; i < n_here * MW; i += 256) block[(i / MW) * (MW + 1) + i % MW] = src[i];
    __syncthreads();
    uint32_t *out = rows + (int64_t)tile_local * (M + 2) * tw;
    const bool lo_ok = nb * 2 < tw, hi_ok = nb * 2 + 1 < tw;
    for (int j = wave; j < MW; j += 4) {
        const uint32_t word = lane < n_here ? block[lane * (MW + 1) + j] : 0u;
        // each half of the wave transposes its 32 slots x 32 bits: lane b of a half holds one word of row 32 j + b
        const uint32_t column = tile_transpose32(word, lane);
        const int p = j * 32 + (lane & 31);
        if (p < M && (lane < 32 ? lo_ok : hi_ok)) out[(int64_t)p * tw + nb * 2 + (lane >> 5)] = column;
    }
    if (wave == 0) {
        const int pos = nb * 64 + lane;
        const int used = tg.slot_words == 0 ? tw : tg.gpt * tg.slot_words;
        const int gj = pos / tg.slot_bits, n = pos - gj * tg.slot_bits;
        const int64_t g = (int64_t)(tile0 + tile_local) * tg.gpt + gj;
        const bool empty = pos < slots && n == 0 && gj < tg.gpt && g < G && n_nodes[g] == 0u;
        const unsigned long long e = __ballot(empty);
        if (lane == 0) {
            if (lo_ok) {
                out[(int64_t)M * tw + nb * 2] = nb * 2 < used ? 0xFFFFFFFFu : 0u;
                out[(int64_t)(M + 1) * tw + nb * 2] = (uint32_t)e;
            }
            if (hi_ok) {
                out[(int64_t)M * tw + nb * 2 + 1] = nb * 2 + 1 < used ? 0xFFFFFFFFu : 0u;
                out[(int64_t)(M + 1) * tw + nb * 2 + 1] = (uint32_t)(e >> 32);
            }
        }
    }
}

// The three steps above for one graph per workgroup with the vectors in LDS (no sent / got in
// global memory, no global atomics): tiles of whole-word slots, M a multiple of 32, and a graph's
// vectors small enough - 2 * slot_bits * (MW | 1) words of LDS.  grid (graphs per tile,
// tiles of the launch), 1,024 threads.
//   1. sent[slot] |= hypervector bits of every clause true at the slot (LDS atomics)
//   2. got[destination] |= rotate(sent[slot], edge type) along every out-edge (LDS atomics)
//   3. got turned literal-major, 64 slots at a time (two 32 x 32 bit transpositions across the
//      lanes); a wave collects 32 rows in LDS (in
//      the space of sent, which is no longer needed) and writes them whole: rows[tile][M + 2][tw],
//      the graph's words of each; plus the all-ones row and the row of graphs without nodes.
// The workgroup of a tile's last graph also clears the words past the last slot of every row.
constexpr int TILE_FUSED_MESSAGES_BLOCK = 1024;

inline size_t tile_fused_messages_lds_bytes(const TileGeom &g, int MW) {
    // vectors are MW | 1 words apart plus one word per 32 slots: lanes on neighbouring slots hit different
    // banks, and so do lanes on the same bit of different words of a truth row (32 slots apart)
    return 2 * ((size_t)g.slot_bits * (MW | 1) + (size_t)g.slot_words) * 4;
}

__global__ __launch_bounds__(TILE_FUSED_MESSAGES_BLOCK) void k_tile_messages_fused(
    const uint32_t *__restrict__ bitmap, int C, TileGeom tg, int tile0, int G, int M, int MW,
    const uint32_t *__restrict__ bit_start, const uint32_t *__restrict__ bit_clauses, const uint32_t *__restrict__ node_index,
    const uint32_t *__restrict__ n_nodes, const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
    const uint32_t *__restrict__ edge, int has_edges, uint32_t *__restrict__ rows) {
    extern __shared__ uint32_t lds[];
    constexpr int NT = TILE_FUSED_MESSAGES_BLOCK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gj = blockIdx.x, tile_local = blockIdx.y;
    const int tw = tg.tw, sw = tg.slot_words, slots = tg.slot_bits, MWP = MW | 1;
    const int VEC = slots * MWP + sw;   // slot n's vector starts at n * MWP + n / 32
    uint32_t *sent = lds;
    uint32_t *got = lds + VEC;
    const int64_t g = (int64_t)(tile0 + tile_local) * tg.gpt + gj;
    const int nodes = g < G ? (int)n_nodes[g] : 0;
    const int w_first = gj * sw;        // the graph's first word of a tile row
    uint32_t *out = rows + (int64_t)tile_local * (M + 2) * tw;

    // 1. what every node slot sends: a half-wave takes 32 message bits and up to 8 words of the graph's
    // truth rows at a time (lane = bit: the OR of the truth words of the bit's clauses), transposes,
    // and lane = node stores word j of its vector - each word once, no atomics.  A lane's work is a chain
    // of dependent reads (where the bit's clauses start, which they are, their truth words): the index
    // and the graph's truth rows are first copied into the space of `got`, which is not needed yet, when
    // they fit there, so that the chain runs on LDS.
    if (nodes > 0) {
        constexpr int WB = MESSAGE_WORDS_AT_ONCE;
        const uint32_t *truth = bitmap + (int64_t)tile_local * C * tw + w_first;
        const int used = (nodes + 31) >> 5;  // words of a truth row that can hold a true node
        const uint32_t n_listed = bit_start[M];  // (clause, bit) pairs in the index
        // (staged rows an odd number of words apart: the lanes of a half-wave read words of different clauses)
        const int ts = used | 1;
        const bool staged = (size_t)(M + 1) + n_listed + (size_t)C * ts <= (size_t)VEC;
        uint32_t *s_start = got, *s_clauses = got + (M + 1), *s_truth = s_clauses + n_listed;
        if (staged) {
            for (int i = tid; i <= M; i += NT) s_start[i] = bit_start[i];
            for (uint32_t i = tid; i < n_listed; i += NT) s_clauses[i] = bit_clauses[i];
            // (half a wave per clause and trip: no division to find an element's clause and word)
            for (int c = tid >> 5; c < C; c += NT / 32)
                for (int w = tid & 31; w < used; w += 32) s_truth[c * ts + w] = truth[(int64_t)c * tw + w];
            __syncthreads();
        }
        const int hl = lane & 31, half = lane >> 5;
        const int blocks_w = (used + WB - 1) / WB, tasks = MW * blocks_w;
        for (int t0 = wave * 2; t0 < tasks; t0 += NT / 32) {
            const int t = t0 + half;
            const bool valid = t < tasks;
            const int j = valid ? t / blocks_w : 0, wl0 = valid ? (t - j * blocks_w) * WB : 0;
            const int n_words = valid ? (used - wl0 < WB ? used - wl0 : WB) : 0;
            uint32_t word[WB];
            // (two calls, so that the copies are read with LDS instructions and not through generic pointers)
            if (staged)
                message_bit_words(s_truth + wl0, ts, n_words, s_start, s_clauses, j * 32 + hl, M, word);
            else
                message_bit_words(truth + wl0, tw, n_words, bit_start, bit_clauses, j * 32 + hl, M, word);
#pragma unroll
            for (int u = 0; u < WB; ++u) {
                const uint32_t column = tile_transpose32(word[u], lane);
                if (u < n_words) sent[((wl0 + u) * 32 + hl) * MWP + (wl0 + u) + j] = column;
            }
        }
    }
    __syncthreads();
    for (int i = tid; i < VEC; i += NT) got[i] = 0u;  // (every word of sent that is read has been stored)
    __syncthreads();

    // 2. along the edges: bit p of what arrives is bit (p - type) mod M of what was sent
    // (one thread per node: its edge list is two dependent memory round trips, paid once for all
    // the vector words)
    if (has_edges && nodes > 0) {
        const int64_t row0 = node_index[g];
        for (int n = tid; n < nodes; n += NT) {
            const uint32_t *v = sent + n * MWP + (n >> 5);
            const uint32_t ne = n_edges[row0 + n];
            const uint2 *out_edges = reinterpret_cast<const uint2 *>(edge) + edge_index[row0 + n];
            // (vectors of at most 16 words are read once, into registers, for all the node's edges)
            constexpr int IN_REGISTERS = 16;
            uint32_t mine[IN_REGISTERS];
#pragma unroll
            for (int j = 0; j < IN_REGISTERS; ++j) mine[j] = MW <= IN_REGISTERS && j < MW ? v[j] : 0u;
            const uint32_t last = v[MW - 1];
            for (uint32_t e0 = 0; e0 < ne; e0 += 4) {
                uint2 pair[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) pair[u] = e0 + u < ne ? out_edges[e0 + u] : make_uint2(0u, 0u);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (e0 + u >= ne) break;
                    const uint32_t dst = pair[u].x, shift = pair[u].y % (uint32_t)M;
                    const int q = (int)(shift >> 5), r = (int)(shift & 31u);
                    uint32_t *to = got + dst * MWP + (dst >> 5);
                    if (MW <= IN_REGISTERS) {
                        int at = q;  // the word that word 0 of the vector goes to
                        const uint32_t down = 32u - (uint32_t)r;  // (word j, word j - 1) moved down by 32 - r: one 64-bit shift
#pragma unroll
                        for (int j = 0; j < IN_REGISTERS; ++j) {
                            if (j < MW) {
                                const uint32_t below = j == 0 ? last : mine[j > 0 ? j - 1 : 0];
                                const uint32_t word = (uint32_t)((((unsigned long long)mine[j] << 32) | below) >> down);
                                if (word) atomicOr(&to[at], word);
                                at = at + 1 == MW ? 0 : at + 1;
                            }
                        }
                    } else {
                        int a = (int)((MW - q) % MW);  // word of v that feeds word 0
                        for (int j = 0; j < MW; ++j) {
                            const int below = a == 0 ? MW - 1 : a - 1;
                            const uint32_t word = r ? (v[a] << r) | (v[below] >> (32 - r)) : v[a];
                            if (word) atomicOr(&to[j], word);
                            a = a + 1 == MW ? 0 : a + 1;
                        }
                    }
                }
            }
        }
    }
    __syncthreads();

    // 3. literal-major rows: wave v turns vector words v, v + 16, ... (32 rows each) and writes
    // the graph's words of those rows; its 32 x sw words of staging live where sent was
    const int pack_waves = MW < NT / 64 ? MW : NT / 64;
    if (wave < pack_waves) {
        // (rows an odd number of words apart where there is room: the 32 lanes that store a column of 32 rows
        // then hit 32 banks, not 2)
        const int ss = pack_waves * 32 * (sw | 1) <= VEC ? sw | 1 : sw;
        uint32_t *stage = sent + wave * 32 * ss;  // [32 rows][ss]
        for (int j = wave; j < MW; j += pack_waves) {
            for (int nb = 0; nb * 2 < sw; ++nb) {
                const int slot = nb * 64 + lane;
                const uint32_t word = slot < slots ? got[slot * MWP + (slot >> 5) + j] : 0u;
                // lanes 0..31 and 32..63 each transpose their 32 x 32 bits: lane b of a half ends up
                // with bit b of the half's 32 slots, i.e. one word of row 32 j + b
                const uint32_t column = tile_transpose32(word, lane);
                if (nb * 2 + (lane >> 5) < sw) stage[(lane & 31) * ss + nb * 2 + (lane >> 5)] = column;
            }
            // (a wave's LDS writes are visible to its own later reads: same wave, in order)
            if (sw <= 32) {  // two rows per trip, a half-wave each
                const int w = lane & 31;
                for (int r = lane >> 5; r < 32; r += 2)
                    if (w < sw) out[(int64_t)(j * 32 + r) * tw + w_first + w] = stage[r * ss + w];
            } else {
                for (int r = 0; r < 32; ++r)
                    for (int w = lane; w < sw; w += 64) out[(int64_t)(j * 32 + r) * tw + w_first + w] = stage[r * ss + w];
            }
        }
    }
    // the all-ones row and the row of graphs without nodes (kernels.py:443-466,505-527 leave every
    // clause true for such a graph at every layer, which the message literals must not undo)
    for (int w = tid; w < sw; w += NT) {
        out[(int64_t)M * tw + w_first + w] = 0xFFFFFFFFu;
        out[(int64_t)(M + 1) * tw + w_first + w] = (w == 0 && g < G && nodes == 0) ? 1u : 0u;
    }
    // words past the tile's last slot
    if (gj == tg.gpt - 1) {
        const int from = tg.gpt * sw, extra = tw - from;
        for (int i = tid; i < (M + 2) * extra; i += NT) {
            const int r = i / extra, w = i - r * extra;
            out[(int64_t)r * tw + from + w] = 0u;
        }
    }
}

// One layer of clause evaluation for one tile per workgroup.
//
// Layer 0 (ROWS_STAGED / ROWS_GLOBAL): a clause's truth over the tile's node
// slots is the AND of the node-type row and the rows of its included literals
// (kernels.py:443-466).  Message layers (ROWS_MESSAGES): the layer's message
// rows (k_tile_*_messages below; row p has the bit of node slot n set iff some
// clause that is true at a neighbour s with an edge s -> n of type t has
// (h + t) mod M == p for one of its hypervector bits h, kernels.py:565-588; the
// negated message literal p + M is the complement of row p) are staged in LDS,
// and a clause's truth is its previous truth AND the rows of its included
// message literals (kernels.py:505-527).
//
// A wave owns a clause at a time.  The clause's row list is wave-uniform: on layer 0
// its first 32 entries arrive by scalar loads issued while the previous clause is
// being evaluated; on message layers, whose rows are in LDS, the lists come by
// vector loads through a few LDS words of the wave's own (see evaluate_listed).
// Lane L holds words [L*LW, (L+1)*LW) of the running AND; after every 8 (16) rows a
// clause that is false at every node slot of the tile is done.
//
// LAST: the clause's weights are added to the class sums of the graphs where it
// is true at some node (kernels.py:297-315) and no bitmap is written; otherwise
// the truth row goes to `bitmap`.
template <int NWAVES, int LW, int SRC, bool LAST>
__global__ __launch_bounds__(NWAVES * 64) void k_tile_layer(TileLayerArgs a) {
    extern __shared__ uint32_t lds[];
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, C = a.C, K = a.K;
    constexpr int NT = NWAVES * 64;
    const int n_rows_lds = SRC == ROWS_STAGED ? tg.rows : SRC == ROWS_MESSAGES ? a.M + 2 : 0;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)n_rows_lds * tw + TILE_LDS_PAD_WORDS);
    const int tile = a.tile0 + blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint32_t *bitmap = a.bitmap + (int64_t)blockIdx.x * C * tw;  // this tile's truth rows

    if (SRC == ROWS_STAGED || SRC == ROWS_MESSAGES) {  // rows -> LDS, 16 bytes per thread and trip, several loads in flight
        const uint4 *src = reinterpret_cast<const uint4 *>(
            SRC == ROWS_STAGED ? a.tiles + (int64_t)tile * tg.rows * tw
                               : a.message_rows + (int64_t)blockIdx.x * n_rows_lds * tw);
        uint4 *dst = reinterpret_cast<uint4 *>(bt);
        const int n4 = (n_rows_lds * tw) >> 2;  // tw is a multiple of 4
        for (int i = tid; i < n4; i += NT * 4) {
            uint4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int at = i + u * NT;
                v[u] = at < n4 ? src[at] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int at = i + u * NT;
                if (at < n4) dst[at] = v[u];
            }
        }
    }
    for (int i = tid; i < TILE_LDS_PAD_WORDS + tg.gpt * K; i += NT) bt[(size_t)n_rows_lds * tw + i] = 0;
    __syncthreads();

    // Lanes past the row width: their running AND starts at 0 and stays 0.  In LDS they read the
    // words after the row (inside the allocation) so that they fall on banks no other lane of
    // the access uses; in global memory they read the row's first words.
    const bool active = lane * LW < tw;
    const char *col = SRC == ROWS_GLOBAL
                          ? reinterpret_cast<const char *>(a.tiles + (int64_t)tile * tg.rows * tw + (active ? lane * LW : 0))
                          : reinterpret_cast<const char *>(bt + lane * LW);

    // lane p < gpt*K adds weight k = p % K to graph j = p / K of the tile
    const int pairs = tg.gpt * K;
    const int my_j = lane / K, my_k = lane - my_j * K;
    const bool pair_lane = LAST && tg.slot_words > 0 && lane < pairs;
    const int my_shift = (lane < tg.gpt ? lane : 0) * tg.lanes_per_graph;
    const unsigned long long slot_lanes = tg.lanes_per_graph >= 64 ? ~0ull : (1ull << tg.lanes_per_graph) - 1ull;

    auto any_bit = [](const LaneWords<LW> &x) {
        uint32_t m = x.w[0];
#pragma unroll
        for (int u = 1; u < LW; ++u) m |= x.w[u];
        return m != 0;
    };
    // acc &= the rows of entries e[from .. 7] of an 8-entry block (their complements: a block is all of one kind)
    auto and_block = [&](LaneWords<LW> &acc, const uint32_t *e, int from, bool complements) {
        LaneWords<LW> r[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i >= from) r[i].load(col + e[i]);
        if (SRC == ROWS_MESSAGES && complements) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i >= from)
#pragma unroll
                    for (int u = 0; u < LW; ++u) acc.w[u] &= ~r[i].w[u];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i >= from)
#pragma unroll
                    for (int u = 0; u < LW; ++u) acc.w[u] &= r[i].w[u];
        }
    };

    // slot bit 0 of the graphs without nodes (message layers)
    LaneWords<LW> empties;
#pragma unroll
    for (int u = 0; u < LW; ++u) empties.w[u] = 0u;
    bool any_empty = false;
    if (SRC == ROWS_MESSAGES) {
        if (active) empties.load(col + (size_t)(a.M + 1) * tw * 4);
        any_empty = __ballot(any_bit(empties)) != 0;
    }

    // What a clause's truth row `acc` adds to the class sums, or the row itself.  `alive`: the clause was true
    // somewhere before this layer.
    auto finish = [&](LaneWords<LW> &acc, bool alive, int my_weight, const int32_t *weights_of_clause,
                      const LaneWords<LW> &truth_in, char *truth_out) {
        if (SRC == ROWS_MESSAGES && any_empty) {
#pragma unroll
            for (int u = 0; u < LW; ++u) acc.w[u] |= truth_in.w[u] & empties.w[u];
        }
        if (!LAST) {
            if (active && (SRC != ROWS_MESSAGES || alive)) acc.store(truth_out);  // a dead row is already all zero in place
            return;
        }
        const unsigned long long nz = alive ? __ballot(any_bit(acc)) : 0ull;
        if (nz == 0) return;
        if (tg.slot_words > 0) {
            // graph j owns lanes [j*lanes_per_graph, (j+1)*lanes_per_graph)
            const unsigned long long gm = __ballot(lane < tg.gpt && ((nz >> my_shift) & slot_lanes) != 0);
            if (pair_lane && ((gm >> my_j) & 1ull)) atomicAdd(&sums[lane], my_weight);
            for (int p = lane + 64; p < pairs; p += 64) {
                int j = p / K, k = p - j * K;
                if ((gm >> j) & 1ull) atomicAdd(&sums[p], weights_of_clause[k]);
            }
        } else {
            // several graphs per word: walk the non-empty slots of this lane's words
            const int per_word = 32 / tg.slot_bits;
            const uint32_t slot_mask = (1u << tg.slot_bits) - 1u;  // slot_bits <= 16
#pragma unroll
            for (int u = 0; u < LW; ++u) {
                uint32_t m = acc.w[u];
                while (m) {
                    int sub = (__ffs(m) - 1) / tg.slot_bits;
                    m &= ~(slot_mask << (sub * tg.slot_bits));
                    int j = (lane * LW + u) * per_word + sub;
                    for (int k = 0; k < K; ++k) atomicAdd(&sums[j * K + k], weights_of_clause[k]);
                }
            }
        }
    };

    // `truth_in` is the clause's truth from the previous layer (message layers only)
    auto evaluate = [&](const Chunk32 &head, const uint32_t *list, const int32_t *weights_of_clause,
                        const LaneWords<LW> &truth_in, char *truth_out) {
        const int my_weight = pair_lane ? weights_of_clause[my_k] : 0;  // needed only if the clause fires
        const int plain = (int)(head.v[0] & 0xFFFFu);  // blocks of rows; the blocks after them: rows to complement
        const int nb = plain + (int)(head.v[0] >> 16);
        LaneWords<LW> acc;
        bool alive = true;
        if (SRC == ROWS_MESSAGES) {
            acc = truth_in;
            alive = __ballot(any_bit(acc)) != 0;
        } else {
#pragma unroll
            for (int u = 0; u < LW; ++u) acc.w[u] = active ? 0xFFFFFFFFu : 0u;
        }
        if (alive) {
            and_block(acc, head.v, 1, false);  // (block 0 starts with the header and is never of the second kind)
            // stop as soon as the clause is false at every node slot of the tile
            if (nb > 1 && __ballot(any_bit(acc)) != 0) {
                // entries past the first chunk, 16 at a time, requested one step before they are needed
                const Chunk16 *tp = reinterpret_cast<const Chunk16 *>(list) + 2;
                Chunk16 tail = *tp;
                and_block(acc, head.v + 8, 0, 1 >= plain);
                if (nb > 2 && __ballot(any_bit(acc)) != 0) {
                    and_block(acc, head.v + 16, 0, 2 >= plain);
                    if (nb > 3 && __ballot(any_bit(acc)) != 0) {
                        and_block(acc, head.v + 24, 0, 3 >= plain);
                        for (int j = 4; j < nb && __ballot(any_bit(acc)) != 0; j += 2) {
                            const Chunk16 ahead = *++tp;
                            and_block(acc, tail.v, 0, j >= plain);
                            if (j + 1 < nb && __ballot(any_bit(acc)) != 0) and_block(acc, tail.v + 8, 0, j + 1 >= plain);
                            tail = ahead;
                        }
                    }
                }
            }
        }
        finish(acc, alive, my_weight, weights_of_clause, truth_in, truth_out);
    };

    // The same for a message layer with the clause's list in this wave's LDS.  A list that comes in by scalar loads
    // is waited for with the counter that the row reads from LDS use as well, and scalar loads return in no fixed
    // order: every wait for a row would also wait for the chunk of the list requested ahead, so nothing is hidden.
    // Here lane l brings entries l, 64 + l, ... of the lists of 8 clauses along with their truth rows (vector loads,
    // a counter of their own), a clause's entries are put into LDS when its turn comes, and the walk reads them back
    // a block ahead of the rows (LDS returns in order): the four lanes of every quad read entries 0..3 and 4..7 of
    // the block, and entry i reaches all lanes inside the add that forms the row's address (quad broadcast).
    constexpr int LIST_REGS = TILE_LIST_ENTRIES / 64;
    // (the registers that the layer's longest list needs are requested for every clause, alive or not)
    const int list_regs = SRC == ROWS_MESSAGES && a.lists_in_lds ? (int)((*a.longest_list + 63u) >> 6) : 0;
    uint32_t *my_list = lds + (size_t)n_rows_lds * tw + TILE_LDS_PAD_WORDS + (size_t)tg.gpt * K + wave * TILE_LIST_LDS_WORDS;
    auto evaluate_listed = [&](const uint32_t (&entries)[LIST_REGS], int plain, int nb, const int32_t *weights_of_clause,
                               const LaneWords<LW> &truth_in, char *truth_out) {
        const int my_weight = pair_lane ? weights_of_clause[my_k] : 0;
        const uint32_t ones_entry = (uint32_t)a.M * (uint32_t)tw * 4u;  // in the place of the header
#pragma unroll
        for (int k = 0; k < LIST_REGS; ++k)
            if (k * 64 < nb * 8) my_list[k * 64 + lane] = k == 0 && lane == 0 ? ones_entry : entries[k];
        LaneWords<LW> acc = truth_in;
        bool alive = true;
        const uint32_t *quad_entry = my_list + (lane & 3);
        auto block_of = [&](uint32_t lo, uint32_t hi, uint32_t (&e)[8]) {
            e[0] = (uint32_t)__builtin_amdgcn_mov_dpp((int)lo, 0x00, 0xF, 0xF, true);
            e[1] = (uint32_t)__builtin_amdgcn_mov_dpp((int)lo, 0x55, 0xF, 0xF, true);
            e[2] = (uint32_t)__builtin_amdgcn_mov_dpp((int)lo, 0xAA, 0xF, 0xF, true);
            e[3] = (uint32_t)__builtin_amdgcn_mov_dpp((int)lo, 0xFF, 0xF, 0xF, true);
            e[4] = (uint32_t)__builtin_amdgcn_mov_dpp((int)hi, 0x00, 0xF, 0xF, true);
            e[5] = (uint32_t)__builtin_amdgcn_mov_dpp((int)hi, 0x55, 0xF, 0xF, true);
            e[6] = (uint32_t)__builtin_amdgcn_mov_dpp((int)hi, 0xAA, 0xF, 0xF, true);
            e[7] = (uint32_t)__builtin_amdgcn_mov_dpp((int)hi, 0xFF, 0xF, 0xF, true);
        };
        // blocks [from, to), all of one kind, two at a time (16 rows in flight, one test for an all-zero row)
        auto walk = [&](int from, int to, bool complements) {
            int b = from;
            uint32_t lo0 = quad_entry[8 * b], hi0 = quad_entry[8 * b + 4];
            uint32_t lo1 = quad_entry[8 * b + 8], hi1 = quad_entry[8 * b + 12];
            for (; b + 1 < to && alive; b += 2) {
                const uint32_t n_lo0 = quad_entry[8 * b + 16], n_hi0 = quad_entry[8 * b + 20];
                const uint32_t n_lo1 = quad_entry[8 * b + 24], n_hi1 = quad_entry[8 * b + 28];
                uint32_t e0[8], e1[8];
                block_of(lo0, hi0, e0);
                block_of(lo1, hi1, e1);
                LaneWords<LW> r[16];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    r[i].load(col + e0[i]);
                    r[8 + i].load(col + e1[i]);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i)
#pragma unroll
                    for (int u = 0; u < LW; ++u) acc.w[u] &= complements ? ~r[i].w[u] : r[i].w[u];
                alive = __ballot(any_bit(acc)) != 0;
                lo0 = n_lo0;
                hi0 = n_hi0;
                lo1 = n_lo1;
                hi1 = n_hi1;
            }
            if (b < to && alive) {  // an odd block at the end
                uint32_t e0[8];
                block_of(lo0, hi0, e0);
                and_block(acc, e0, 0, complements);
                alive = __ballot(any_bit(acc)) != 0;
            }
        };
        walk(0, plain, false);
        if (alive && nb > plain) walk(plain, nb, true);
        finish(acc, true, my_weight, weights_of_clause, truth_in, truth_out);
    };

    if (SRC == ROWS_MESSAGES) {
        // Message layers: many clauses are already false at every node slot of the tile.  A wave reads
        // the truth rows of 8 of its clauses at once, and with them the first entries of their lists,
        // and evaluates only the clauses that are still true somewhere.
        constexpr int GROUP = 8;
        // (every lane loads, from an address that is always valid - a clause past the last one repeats the wave's
        // first, a lane past the row or the list reads its first word - and what must not count is dropped
        // afterwards: no branch around any load, pointers that step by additions)
        const int64_t truth_step = (int64_t)NWAVES * tw, list_step = (int64_t)NWAVES * a.stride;
        const int my_word = active ? lane * LW : 0;
        int my_entry[LIST_REGS];
#pragma unroll
        for (int k = 0; k < LIST_REGS; ++k) my_entry[k] = k * 64 + lane < a.stride ? k * 64 + lane : 0;
        for (int c0 = wave; c0 < C; c0 += GROUP * NWAVES) {
            LaneWords<LW> t[GROUP];
            uint32_t entries[GROUP][LIST_REGS];
            const uint32_t *truth_of = bitmap + (int64_t)c0 * tw, *list_of = a.lists + (int64_t)c0 * a.stride;
#pragma unroll
            for (int g = 0; g < GROUP; ++g) {
                const bool there = c0 + g * NWAVES < C;
                const uint32_t *truth_row = there ? truth_of + g * truth_step : truth_of;
                const uint32_t *list = there ? list_of + g * list_step : list_of;
                t[g].load(reinterpret_cast<const char *>(truth_row + my_word));
#pragma unroll
                for (int k = 0; k < LIST_REGS; ++k) {
                    entries[g][k] = 0u;
                    if (k < list_regs) entries[g][k] = list[my_entry[k]];
                }
            }
#pragma unroll
            for (int g = 0; g < GROUP; ++g)
                if (!active || c0 + g * NWAVES >= C)
#pragma unroll
                    for (int u = 0; u < LW; ++u) t[g].w[u] = 0u;
            auto one_clause = [&](int c, const LaneWords<LW> &truth_in, const uint32_t (&mine)[LIST_REGS]) {
                const uint32_t *list = a.lists + (int64_t)c * a.stride;
                const int32_t *weights_of_clause = LAST ? a.wt + (int64_t)c * K : nullptr;
                char *truth_out = reinterpret_cast<char *>(bitmap + (int64_t)c * tw + (active ? lane * LW : 0));
                if (a.lists_in_lds) {
                    const uint32_t header = (uint32_t)__builtin_amdgcn_readlane((int)mine[0], 0);
                    const int plain = (int)(header & 0xFFFFu), nb = plain + (int)(header >> 16);
                    if (nb * 8 <= TILE_LIST_ENTRIES) {
                        evaluate_listed(mine, plain, nb, weights_of_clause, truth_in, truth_out);
                        return;
                    }
                }
                const Chunk32 head = *reinterpret_cast<const Chunk32 *>(list);
                evaluate(head, list, weights_of_clause, truth_in, truth_out);
            };
            if (LAST) {
                // (with the scoring in it the evaluation is long: one copy in the instruction cache, the clause's
                // registers picked out of the 8, measured faster than 8 copies; without it the other way round)
                uint32_t alive_of_8 = 0u;  // (a clause that is false everywhere costs no more than this test)
#pragma unroll
                for (int g = 0; g < GROUP; ++g)
                    if (c0 + g * NWAVES < C && __ballot(any_bit(t[g])) != 0) alive_of_8 |= 1u << g;
#pragma unroll 1
                for (; alive_of_8 != 0u; alive_of_8 &= alive_of_8 - 1u) {
                    const int g = __builtin_ctz(alive_of_8);
                    LaneWords<LW> truth_in = t[0];
                    uint32_t mine[LIST_REGS];
#pragma unroll
                    for (int k = 0; k < LIST_REGS; ++k) mine[k] = entries[0][k];
#pragma unroll
                    for (int h = 1; h < GROUP; ++h) {
                        if (g == h) {
                            truth_in = t[h];
#pragma unroll
                            for (int k = 0; k < LIST_REGS; ++k) mine[k] = entries[h][k];
                        }
                    }
                    one_clause(c0 + g * NWAVES, truth_in, mine);
                }
            } else {
#pragma unroll
                for (int g = 0; g < GROUP; ++g) {
                    const int c = c0 + g * NWAVES;
                    if (c < C && __ballot(any_bit(t[g])) != 0) one_clause(c, t[g], entries[g]);
                }
            }
        }
    } else {
        // Two clauses per trip so that the chunk fetched ahead never has to be copied.  Pointers step
        // by NWAVES clauses; past the end they stay on the wave's last clause (a valid address whose
        // data is not used).
        // gridDim.y workgroups share the tile's clauses (rows read in place: nothing ties a tile to one)
        const int c_step = NWAVES * (int)gridDim.y, c_first = wave + NWAVES * (int)blockIdx.y;
        const int64_t list_step = (int64_t)c_step * a.stride;
        const int wt_step = c_step * K;
        const int64_t truth_step = (int64_t)c_step * tw * 4;
        const int first = c_first < C ? c_first : 0;
        const uint32_t *list_a = a.lists + (int64_t)first * a.stride;
        const int32_t *wt_a = LAST ? a.wt + (int64_t)first * K : nullptr;
        char *truth_a = reinterpret_cast<char *>(bitmap + (int64_t)first * tw + (active ? lane * LW : 0));
        Chunk32 ca = *reinterpret_cast<const Chunk32 *>(list_a);
        LaneWords<LW> none;
#pragma unroll
        for (int u = 0; u < LW; ++u) none.w[u] = 0u;
        for (int c = c_first; c < C; c += 2 * c_step) {
            const bool has_b = c + c_step < C;
            const uint32_t *list_b = has_b ? list_a + list_step : list_a;
            const int32_t *wt_b = LAST ? (has_b ? wt_a + wt_step : wt_a) : nullptr;
            char *truth_b = has_b ? truth_a + truth_step : truth_a;
            const Chunk32 cb = *reinterpret_cast<const Chunk32 *>(list_b);
            evaluate(ca, list_a, wt_a, none, truth_a);
            const bool has_a = c + 2 * c_step < C;
            list_a = has_a ? list_b + list_step : list_b;
            if (LAST) wt_a = has_a ? wt_b + wt_step : wt_b;
            truth_a = has_a ? truth_b + truth_step : truth_b;
            ca = *reinterpret_cast<const Chunk32 *>(list_a);
            if (has_b) evaluate(cb, list_b, wt_b, none, truth_b);
        }
    }
    if (!LAST) return;
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NT) {
        int64_t g = g0 + i / K;
        if (g >= a.first_graph && g < (int64_t)a.first_graph + a.n_graphs) {
            // workgroups that share a tile add their shares (the host cleared the sums)
            if (gridDim.y > 1) {
                if (sums[i] != 0) atomicAdd(&a.class_sum[(g - a.first_graph) * K + (i % K)], sums[i]);
            } else {
                a.class_sum[(g - a.first_graph) * K + (i % K)] = sums[i];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Layer 0 in two phases, for tiles of whole-word graph slots whose nodes have
// few literal words (LA a multiple of 4, at most 16).
//
// Phase 1 ANDs the node-type row and the rows of the clause's 14 rarest
// included literals, which leaves very few candidate node slots; phase 2 tests
// each candidate against the clause's whole include mask on the node's own
// literal words (X, node-major, as kernels.py:443-466 reads it):
// the clause is true at the node iff (include & ~X[node]) == 0.  The result is
// the same truth row as ANDing every included literal's row.
//
// Compiled clause: 16 entries of 16 bits - entry 0 = rows in use (type row +
// literals, at most 15) | needs-phase-2 << 8; entries 1..15 = row offsets in
// units of 16 bytes, unused ones pointing at the all-ones row - followed by the
// LA words of the include mask.

constexpr int TWO_PHASE_WALK_FROM = 6;  // slots a lane has left besides its first from which a clause's rows are all walked instead

struct alignas(32) Packed8 {
    uint32_t v[8];
};
template <int N>
struct alignas(16) Words {
    uint32_t v[N];
};

__global__ void k_compile_clauses_two_phase(const uint32_t *__restrict__ bank, int C, int chunks, int B,
                                            uint32_t filter, int literals, int n_types, int type_base_row,
                                            int ones_row, int tw, const uint32_t *__restrict__ order,
                                            uint32_t *__restrict__ records, int record_words, int K,
                                            const int32_t *__restrict__ weights, int32_t *__restrict__ wt) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (c >= C) return;
    const uint32_t row16 = (uint32_t)tw >> 2;  // a row in units of 16 bytes (tw is a multiple of 4)
    uint32_t *rec = records + (int64_t)c * record_words;
    uint16_t *e = reinterpret_cast<uint16_t *>(rec);
    const uint32_t *inc = bank + (int64_t)c * chunks * B + (B - 1);
    if (lane == 0) e[1] = (uint16_t)((uint32_t)(type_base_row + c % n_types) * row16);
    int n = 2;
    for (int r0 = 0; r0 < literals; r0 += 64) {
        int r = r0 + lane;
        uint32_t lit = r < literals ? (order ? order[r] : (uint32_t)r) : 0u;
        uint32_t w = lit >> 5;
        uint32_t word = inc[(int64_t)w * B];
        if ((int)w == chunks - 1) word &= filter;
        bool included = r < literals && ((word >> (lit & 31)) & 1u);
        unsigned long long mask = __ballot(included);
        int at = n + __popcll(mask & ((1ull << lane) - 1ull));
        if (included && at < 16) e[at] = (uint16_t)(lit * row16);
        n += __popcll(mask);
    }
    for (int i = n + lane; i < 16; i += 64) e[i] = (uint16_t)((uint32_t)ones_row * row16);
    if (lane == 0) e[0] = (uint16_t)((n > 16 ? 15 : n - 1) | (n > 16 ? 0x100 : 0));
    for (int w = lane; w < chunks; w += 64) {
        uint32_t word = inc[(int64_t)w * B];
        if (w == chunks - 1) word &= filter;
        rec[8 + w] = word;
    }
    if (weights)
        for (int k = lane; k < K; k += 64) wt[(int64_t)c * K + k] = weights[(int64_t)k * C + c];
}

// The two phases of a clause are software-pipelined: a wave issues the phase-2 loads of one clause
// (each lane the literal words of its first surviving node slot), runs phase 1 of its next clause
// while they are in flight, and only then finishes the first.  Lanes with more than one surviving
// slot test the others in a loop afterwards (rare once 14 literals have been applied).
template <int NWAVES, int LW, int LA4, bool LAST, bool FULL>
__global__ __launch_bounds__(NWAVES * 64) void k_tile_two_phase(TileLayerArgs a) {
    extern __shared__ uint32_t lds[];
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, C = a.C, K = a.K;
    constexpr int NT = NWAVES * 64;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)tg.rows * tw + TILE_LDS_PAD_WORDS);
    const int tile = a.tile0 + blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint32_t *bitmap = a.bitmap + (int64_t)blockIdx.x * C * tw;

    {  // tile -> LDS
        const uint4 *src = reinterpret_cast<const uint4 *>(a.tiles + (int64_t)tile * tg.rows * tw);
        uint4 *dst = reinterpret_cast<uint4 *>(bt);
        const int n4 = (tg.rows * tw) >> 2;
        for (int i = tid; i < n4; i += NT * 4) {
            uint4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int at = i + u * NT;
                v[u] = at < n4 ? src[at] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int at = i + u * NT;
                if (at < n4) dst[at] = v[u];
            }
        }
        for (int i = tid; i < TILE_LDS_PAD_WORDS + tg.gpt * K; i += NT) bt[(size_t)tg.rows * tw + i] = 0;
    }
    __syncthreads();

    // FULL: rows are exactly 64 * LW words wide, padded with words that are zero in the node-type
    // rows, so every lane holds real words and no lane needs masking off.
    const bool active = FULL || lane * LW < tw;
    const char *col = reinterpret_cast<const char *>(bt + lane * LW);

    // the graph whose slot this lane's words belong to, and the node of the lane's first bit
    const int lpg = tg.lanes_per_graph;
    const int lane_j = lane / lpg;
    const int64_t lane_g = (int64_t)tile * tg.gpt + lane_j;
    const bool has_graph = active && lane_j < tg.gpt && lane_g < a.G;
    // a graph without nodes keeps its slot bit 0 (every clause is true for it) and has no node to test
    const bool testable = has_graph && a.n_nodes[lane_g] != 0u;
    // byte offset of that node's literal words in X (the host checks that X is smaller than 4 GiB)
    const uint32_t lane_x0 =
        has_graph ? (a.node_index[lane_g] + (uint32_t)(lane - lane_j * lpg) * (LW * 32)) * (LA4 * 16u) : 0u;
    const char *x_base = reinterpret_cast<const char *>(a.X);

    // lane p adds weight k = p % K to graph j = p / K of the tile, for p = lane and p = lane + 64
    const int pairs = tg.gpt * K;
    const int j0 = lane / K, k0 = lane - j0 * K;
    const int j1 = (lane + 64) / K, k1 = lane + 64 - j1 * K;
    const bool pair0 = LAST && lane < pairs, pair1 = LAST && lane + 64 < pairs;
    const uint32_t k0_bytes = pair0 ? k0 * 4u : 0u, k1_bytes = pair1 ? k1 * 4u : 0u;
    const uint32_t shift0 = pair0 ? j0 * lpg : 0, shift1 = pair1 ? j1 * lpg : 0;  // first lane of the pair's graph
    const int my_shift = (lane < tg.gpt ? lane : 0) * lpg;
    const unsigned long long slot_lanes = lpg >= 64 ? ~0ull : (1ull << lpg) - 1ull;

    auto any_bit = [](const LaneWords<LW> &x) {
        uint32_t m = x.w[0];
#pragma unroll
        for (int u = 1; u < LW; ++u) m |= x.w[u];
        return m != 0;
    };
    auto entry_of = [](const Packed8 &rec, int i) { return ((rec.v[i >> 1] >> ((i & 1) * 16)) & 0xFFFFu) << 4; };
    auto and_row = [&](LaneWords<LW> &acc, uint32_t byte_offset) {
        LaneWords<LW> r;
        r.load(col + byte_offset);
#pragma unroll
        for (int u = 0; u < LW; ++u) acc.w[u] &= r.w[u];
    };
    auto violates = [](const Words<4 * LA4> &include, const uint4 *x) {
        uint32_t violated = 0;
#pragma unroll
        for (int q = 0; q < LA4; ++q) {
            const uint4 v = x[q];
            violated |= (include.v[4 * q] & ~v.x) | (include.v[4 * q + 1] & ~v.y) | (include.v[4 * q + 2] & ~v.z) |
                        (include.v[4 * q + 3] & ~v.w);
        }
        return violated != 0;
    };
    // the word set with only `bit` set (bit < 32 * LW)
    auto one_hot = [](uint32_t bit) {
        LaneWords<LW> m;
        if (LW == 1) {
            m.w[0] = 1u << (bit & 31u);
        } else {
#pragma unroll
            for (int h = 0; h < LW / 2; ++h) {
                const unsigned long long v = (LW == 2 || (int)(bit >> 6) == h) ? 1ull << (bit & 63u) : 0ull;
                m.w[2 * h] = (uint32_t)v;
                m.w[2 * h + 1] = (uint32_t)(v >> 32);
            }
        }
        return m;
    };

    struct Pending {
        LaneWords<LW> acc;
        uint4 x[LA4];
        uint32_t bit;            // the node slot this lane has under test (index into its LW words), ~0 if none
        bool live, test;         // wave-uniform: a clause is pending / its phase 2 runs
        unsigned long long nz;   // lanes with a surviving slot after phase 1
        int weight0, weight1;
        const int32_t *weights;
        char *truth_out;
    };

    // Phase 1 and the loads of phase 2.  Every load is issued by all lanes whatever the clause
    // does, so that the number of loads in flight is known when the pending clause is finished.
    auto begin = [&](Pending &p, const Packed8 &rec, const int32_t *weights_of_clause, char *truth_out) {
        p.live = true;
        p.weights = weights_of_clause;
        p.truth_out = truth_out;
        if (LAST) {  // needed only if the clause fires
            const char *wb = reinterpret_cast<const char *>(weights_of_clause);
            p.weight0 = *reinterpret_cast<const int32_t *>(wb + k0_bytes);
            p.weight1 = *reinterpret_cast<const int32_t *>(wb + k1_bytes);
        }
        const uint32_t header = rec.v[0] & 0xFFFFu;
        LaneWords<LW> acc;
#pragma unroll
        for (int u = 0; u < LW; ++u) acc.w[u] = active ? 0xFFFFFFFFu : 0u;
        if ((header & 0xFFu) > 7u) {
#pragma unroll
            for (int i = 1; i < 16; ++i) and_row(acc, entry_of(rec, i));
        } else {
#pragma unroll
            for (int i = 1; i < 8; ++i) and_row(acc, entry_of(rec, i));
        }
        p.nz = __ballot(any_bit(acc));
        p.test = (header & 0x100u) && p.nz != 0;
        // lowest surviving slot of the lane; __ffs(0) - 1 is ~0, which also survives the OR and the min
        uint32_t bit = ~0u;
#pragma unroll
        for (int u = LW - 1; u >= 0; --u) {
            const uint32_t at = (uint32_t)(__ffs(acc.w[u]) - 1) | (uint32_t)(u * 32);
            bit = at < bit ? at : bit;
        }
        p.bit = testable ? bit : ~0u;
        // lanes with nothing to test all read the first node's words (one cache line for the wave)
        const uint32_t x_off = p.bit != ~0u ? lane_x0 + p.bit * (LA4 * 16u) : 0u;
        const uint4 *x = reinterpret_cast<const uint4 *>(x_base + x_off);
#pragma unroll
        for (int q = 0; q < LA4; ++q) p.x[q] = x[q];
        p.acc = acc;
    };

    // The rest of phase 2, then the clause's votes (or its truth row).
    auto finish = [&](Pending &p, const Words<4 * LA4> &include) {
        if (!p.live) return;
        p.live = false;
        LaneWords<LW> acc = p.acc;
        unsigned long long nz = p.nz;
        if (p.test) {
            const bool tested = p.bit != ~0u;
            const bool failed = violates(include, p.x) && tested;
            // the lane's other surviving slots
            const LaneWords<LW> hot = one_hot(p.bit);
            LaneWords<LW> rest;
#pragma unroll
            for (int u = 0; u < LW; ++u) {
                rest.w[u] = acc.w[u] & ~hot.w[u];
                acc.w[u] = failed ? rest.w[u] : acc.w[u];
            }
            if (__ballot(tested && any_bit(rest)) != 0) {
                int others = 0;
#pragma unroll
                for (int u = 0; u < LW; ++u) others += __popc(tested ? rest.w[u] : 0u);
                if (__builtin_expect(__ballot(others >= TWO_PHASE_WALK_FROM) != 0, 0)) {
                    // Phase 1 has left some lane several slots (its literals hold nearly everywhere:
                    // negated ones, mostly), and testing them costs a memory round trip each.  The
                    // rows of ALL the clause's literals are ANDed instead, as k_tile_layer does
                    // (row l belongs to literal l; unused reads take the all-ones row).
                    acc = p.acc;
                    const uint32_t row_bytes = (uint32_t)a.tg.tw * 4u, ones = (uint32_t)(a.tg.rows - 1);
                    uint32_t include_of_lane = 0u;  // lane w holds include word w: one copy of the loop below
#pragma unroll
                    for (int w = 0; w < 4 * LA4; ++w) include_of_lane = lane == w ? include.v[w] : include_of_lane;
#pragma unroll 1
                    for (int w = 0; w < 4 * LA4; ++w) {
                        uint32_t m = __builtin_amdgcn_readlane(include_of_lane, w);
                        while (m) {
                            LaneWords<LW> r[8];
#pragma unroll
                            for (int u = 0; u < 8; ++u) {
                                const uint32_t lit = m ? (uint32_t)(w * 32 + __builtin_ctz(m)) : ones;
                                m &= m - 1u;
                                r[u].load(col + lit * row_bytes);
                            }
#pragma unroll
                            for (int u = 0; u < 8; ++u)
#pragma unroll
                                for (int v = 0; v < LW; ++v) acc.w[v] &= r[u].w[v];
                        }
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < LW; ++u) {
                        uint32_t todo = tested ? rest.w[u] : 0u;
                        while (todo) {
                            const int b = __ffs(todo) - 1;
                            todo &= todo - 1;
                            const uint4 *x =
                                reinterpret_cast<const uint4 *>(x_base + (lane_x0 + (u * 32 + b) * (LA4 * 16u)));
                            if (violates(include, x)) acc.w[u] &= ~(1u << b);
                        }
                    }
                }
            }
            nz = __ballot(any_bit(acc));
        }
        if (!LAST) {
            if (active) acc.store(p.truth_out);
            return;
        }
        if (nz == 0) return;
        // graph j owns lanes [j*lanes_per_graph, (j+1)*lanes_per_graph)
        if (lpg <= 32 && pairs <= 128) {
            const uint32_t m = (uint32_t)slot_lanes;
            if (pair0 && ((uint32_t)(nz >> shift0) & m) != 0) atomicAdd(&sums[lane], p.weight0);
            if (pair1 && ((uint32_t)(nz >> shift1) & m) != 0) atomicAdd(&sums[lane + 64], p.weight1);
        } else {
            const unsigned long long gm = __ballot(lane < tg.gpt && ((nz >> my_shift) & slot_lanes) != 0);
            if (pair0 && ((gm >> j0) & 1ull)) atomicAdd(&sums[lane], p.weight0);
            if (pair1 && ((gm >> j1) & 1ull)) atomicAdd(&sums[lane + 64], p.weight1);
            for (int q = lane + 128; q < pairs; q += 64) {
                int j = q / K, k = q - j * K;
                if ((gm >> j) & 1ull) atomicAdd(&sums[q], p.weights[k]);
            }
        }
    };

    // Clause records: the 8 words of row entries are fetched one clause ahead of phase 1, the
    // include mask at the start of the clause's phase 1 (it is first needed when the clause is
    // finished, one phase 1 later).  Pointers step by NWAVES clauses; past the end they stay on
    // the wave's last clause (a valid address whose data is not used).
    const int64_t rec_step = (int64_t)NWAVES * a.stride;
    const int wt_step = NWAVES * K;
    const int64_t truth_step = (int64_t)NWAVES * tw * 4;
    const int first = wave < C ? wave : 0;
    const uint32_t *rec_a = a.lists + (int64_t)first * a.stride;
    const int32_t *wt_a = LAST ? a.wt + (int64_t)first * K : nullptr;
    char *truth_a = reinterpret_cast<char *>(bitmap + (int64_t)first * tw + (active ? lane * LW : 0));
    Packed8 ea = *reinterpret_cast<const Packed8 *>(rec_a);
    Words<4 * LA4> ma, mb;
    Pending pa, pb;
    pa.live = pb.live = false;
    for (int c = wave; c < C; c += 2 * NWAVES) {
        const bool has_b = c + NWAVES < C;
        const uint32_t *rec_b = has_b ? rec_a + rec_step : rec_a;
        const int32_t *wt_b = LAST ? (has_b ? wt_a + wt_step : wt_a) : nullptr;
        char *truth_b = has_b ? truth_a + truth_step : truth_a;
        ma = *reinterpret_cast<const Words<4 * LA4> *>(rec_a + 8);
        const Packed8 eb = *reinterpret_cast<const Packed8 *>(rec_b);
        begin(pa, ea, wt_a, truth_a);
        finish(pb, mb);
        const bool has_a = c + 2 * NWAVES < C;
        rec_a = has_a ? rec_b + rec_step : rec_b;
        if (LAST) wt_a = has_a ? wt_b + wt_step : wt_b;
        truth_a = has_a ? truth_b + truth_step : truth_b;
        // without a second clause this repeats the first one and drops the result: keeping the
        // sequence of loads the same on every trip lets the waits stay partial
        mb = *reinterpret_cast<const Words<4 * LA4> *>(rec_b + 8);
        ea = *reinterpret_cast<const Packed8 *>(rec_a);
        begin(pb, eb, wt_b, truth_b);
        pb.live = has_b;
        finish(pa, ma);
    }
    finish(pb, mb);
    if (!LAST) return;
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NT) {
        int64_t g = g0 + i / K;
        if (g >= a.first_graph && g < (int64_t)a.first_graph + a.n_graphs)
            a.class_sum[(g - a.first_graph) * K + (i % K)] = sums[i];
    }
}


// ---------------------------------------------------------------------------
// Sharing the tiles of a launch out among the compute units when they do not fill a whole number of
// rounds (477 tiles on 256 CUs: a second round that leaves 35 CUs idle).  The first R * cus tiles
// (R = tiles / cus) are taken whole, one workgroup each.  The (tile, clause) pairs of the remaining
// tiles, tile after tile, are cut into `cus` equal shares; a share lies in one tile or straddles two,
// so it is at most two segments, each a workgroup of its own: 2 * cus more workgroups (some empty).
// Workgroups are handed to the CUs in the order of their numbers as CUs fall free, so the first
// segments come ordered by size, smallest first, and the second segments in the same order of their
// shares - largest first, since the two add up to a share: whoever finishes a short first segment
// finds a long second one next in line, and all finish together.  The table is made, a few entries per
// block, by the launch that compiles the clauses, which also clears the class sums of the graphs of the
// shared tiles, to which their workgroups add.
struct TileSegment {
    int tile_local, c_begin, c_end;
};

constexpr int TILE_SEGMENTS_MAX_SHARES = 1024;

// What the table is made from; cus == 0: no table, one workgroup per tile.
struct SegmentPlan {
    int n_tiles, C, cus, gpt, K, tile0, first_graph, n_graphs;
    TileSegment *segments;  // [tile_segment_count(n_tiles, cus)]
    int32_t *class_sum;     // [n_graphs][K]
};

inline int tile_segment_count(int n_tiles, int cus) { return n_tiles / cus * cus + 2 * cus; }

// Block `block` of `n_blocks` (the blocks of the launch that compiles the clauses: every block does a little of
// this before its clauses, so that the table costs the step no time of its own): its slice of the whole-tile
// entries and of the class sums to clear, and the two segments of the shares block, block + n_blocks, ...
// Share j is pairs [from(j), from(j + 1)) of the remaining tiles' (tile, clause) pairs, from(j) = j * (pairs /
// cus) + min(j, pairs % cus); its place in the table is the rank of its first segment's length among all shares
// (ties by share number), which every block works out for its own shares by counting.  All threads of the block
// must call this (it has barriers); pairs < 2^31 (plan_segments).
__device__ __forceinline__ void tile_segments_part(const SegmentPlan &sp, int block, int n_blocks, int tid, int threads) {
    __shared__ int counted[16];
    const uint32_t C = (uint32_t)sp.C, cus = (uint32_t)sp.cus;
    const int whole = sp.n_tiles / sp.cus * sp.cus, rest = sp.n_tiles - whole;
    for (int b = block * threads + tid; b < whole; b += n_blocks * threads) sp.segments[b] = TileSegment{b, 0, sp.C};
    // the class sums of the graphs of the shared tiles start at zero
    const long long g_lo = (long long)(sp.tile0 + whole) * sp.gpt, g_hi = (long long)(sp.tile0 + sp.n_tiles) * sp.gpt;
    const long long first = sp.first_graph, end = first + sp.n_graphs;
    for (long long i = (g_lo > first ? g_lo : first) * sp.K + block * threads + tid; i < (g_hi < end ? g_hi : end) * sp.K;
         i += (long long)n_blocks * threads)
        sp.class_sum[i - first * sp.K] = 0;
    const uint32_t pairs = (uint32_t)rest * C, base = pairs / cus, extra = pairs % cus;
    auto from_of = [&](uint32_t j) { return j * base + (j < extra ? j : extra); };
    auto first_length = [&](uint32_t j, uint32_t *tile_a, uint32_t *at, uint32_t *length) {
        const uint32_t from = from_of(j);
        *length = from_of(j + 1) - from;
        *tile_a = from / C;
        *at = from - *tile_a * C;
        return *length < C - *at ? *length : C - *at;
    };
    for (uint32_t j = (uint32_t)block; j < cus; j += (uint32_t)n_blocks) {
        uint32_t tile_a, at, length, t, a2, l2;
        const uint32_t len_a = first_length(j, &tile_a, &at, &length);
        int before = 0;
        for (uint32_t k = (uint32_t)tid; k < cus; k += (uint32_t)threads) {
            const uint32_t len_k = first_length(k, &t, &a2, &l2);
            before += len_k < len_a || (len_k == len_a && k < j);
        }
        for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
        __syncthreads();  // (the block's last round has been read)
        if ((tid & 63) == 0) counted[(tid >> 6) & 15] = before;
        __syncthreads();
        if (tid == 0) {
            int rank = 0;
            for (int w = 0; w < (threads + 63) / 64 && w < 16; ++w) rank += counted[w];
            sp.segments[whole + rank] = TileSegment{whole + (int)tile_a, (int)at, (int)(at + len_a)};
            // (empty when the share lies in one tile)
            sp.segments[whole + (int)cus + rank] = TileSegment{whole + (int)tile_a + 1, 0, (int)(length - len_a)};
        }
    }
}

// ---------------------------------------------------------------------------
// The two-phase layer 0 on HALF tiles: LDS holds only the rows of the positive
// literals (plus the node-type rows and the all-ones row), and a negated literal
// l + hv is evaluated as the complement of row l.  That is exact where the data
// set's negated literals are the complements of its positive ones on every node
// (graphs.py:91-98,148-159 build them so; the caller asserts it, GTM_GRAPHS_COMPLEMENTARY)
// and no graph is empty: on node slots past a graph's nodes the complement is 1, but the
// node-type row, which every clause ANDs first, is 0 there.  Half the rows per graph buy
// twice the graphs per tile: the scalar work, the address arithmetic and the phase-2 loads
// of a (clause, tile) pair are spread over twice as many graphs.
//
// Compiled clause, 16 + LA + 4 words: 16 entries of 32 bits, the include words, two more entries.  Entry 0 =
// rows in use (7 or 17) | needs-phase-2 << 8 | positive pairs << 12; the others are rows as
// LDS byte offsets, ready for use (a scalar load puts them in registers): entry 1 = the
// node-type row; then literal rows in PAIRS, 3 or 8 of them (rows 15 and 16 are the two
// entries after the include words): first the pairs of positive
// literals (an odd one out is paired with the all-ones row), then the pairs of negated
// ones (padded with the all-zero words that follow the rows in LDS).  With the signs fixed
// per pair, a pair costs one 3-input bit operation per word of the lane - acc & a & b or
// acc & ~(a | b) - and the clause's pattern (how many positive pairs) selects one of 9
// straight-line variants with a single scalar jump.
// The filter takes the clause's rarest literals, at most 16, as many as fit the pairs: measured on the
// 361-node workload after one epoch, 6 pairs 0.409 ms per 10,000 graphs, 7 pairs 0.358, 8 pairs 0.353 - a
// stronger filter leaves fewer lanes with candidates whose tests wait for memory in the open.

struct alignas(16) Entries16 {
    uint32_t v[16];
};

// Row pairs that phase 1 of the half-tile kernel ANDs for a clause of many literals.  A record is 16 entries (header,
// node-type row, 14 rows), the include words, and the rows past the 14th (4 words kept for them).
constexpr int HALF_BIG_PAIRS = 8;
constexpr int HALF_RECORD_EXTRA_WORDS = 4;

// Index of the lowest set bit, ~0 for 0: what the instruction gives by itself (the compiler's count of trailing
// zeros is either undefined for 0 or comes with a comparison and a select for it).
__device__ __forceinline__ uint32_t lowest_bit_or_ones(uint32_t x) {
    uint32_t r;
    asm("v_ffbl_b32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Last word of a buffer descriptor for plain 32-bit data on this GPU family (raw buffer: byte offsets, range
// checked against the size in bytes).
constexpr int BUFFER_RSRC_FLAGS = 0x00020000;

__global__ void k_compile_clauses_half(const uint32_t *__restrict__ bank, int C, int chunks, int B, uint32_t filter,
                                       int literals, int n_types, int tw, const uint32_t *__restrict__ order,
                                       uint32_t *__restrict__ records, int record_words, int K,
                                       const int32_t *__restrict__ weights, int32_t *__restrict__ wt, SegmentPlan sp) {
    __shared__ uint32_t chosen_of_wave[4][2 + 2 * HALF_BIG_PAIRS + 2];
    if (sp.cus > 0) tile_segments_part(sp, blockIdx.x, gridDim.x, threadIdx.x, blockDim.x);  // which workgroup takes what (see above)
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (c >= C) return;  // whole waves leave; no barrier below
    uint32_t *chosen = chosen_of_wave[(threadIdx.x >> 6) & 3];
    const int hv = literals >> 1;
    const uint32_t row16 = (uint32_t)tw >> 2;  // a row in units of 16 bytes (tw is a multiple of 4)
    const uint32_t ones_row = (uint32_t)(hv + n_types), zero_row = ones_row + 1u;  // the zeroed words after the rows
    uint32_t *rec = records + (int64_t)c * record_words;
    const uint32_t *inc = bank + (int64_t)c * chunks * B + (B - 1);
    // the clause's 16 rarest included literals, in `order`
    int n = 0;
    for (int r0 = 0; r0 < literals; r0 += 64) {
        const int r = r0 + lane;
        const uint32_t lit = r < literals ? order[r] : 0u;
        const uint32_t w = lit >> 5;
        uint32_t word = inc[(int64_t)w * B];
        if ((int)w == chunks - 1) word &= filter;
        const bool included = r < literals && ((word >> (lit & 31)) & 1u);
        const unsigned long long mask = __ballot(included);
        const int at = n + __popcll(mask & ((1ull << lane) - 1ull));
        if (included && at < 2 * HALF_BIG_PAIRS) chosen[at] = lit;
        n += __popcll(mask);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
    int taken = n < 2 * HALF_BIG_PAIRS ? n : 2 * HALF_BIG_PAIRS;
    const uint32_t lit = lane < taken ? chosen[lane] : 0u;
    bool positive = lane < taken && (int)lit < hv, negative = lane < taken && (int)lit >= hv;
    int p = __popcll(__ballot(positive)), q = __popcll(__ballot(negative));
    // 8 pairs hold p positives and q negatives if ceil(p / 2) + ceil(q / 2) <= 8: 16 literals with an
    // odd number of each sign do not fit, and then the least rare of the 16 is left to phase 2
    if (p + q == 2 * HALF_BIG_PAIRS && (p & 1)) {
        --taken;
        if (lane == taken) positive = negative = false;
        p = __popcll(__ballot(positive)), q = __popcll(__ballot(negative));
    }
    const int a = (p + 1) >> 1, b = (q + 1) >> 1;
    const int pairs = a + b <= 3 ? 3 : HALF_BIG_PAIRS;
    const int pos_rank = __popcll(__ballot(positive) & ((1ull << lane) - 1ull));
    const int neg_rank = __popcll(__ballot(negative) & ((1ull << lane) - 1ull));
    // the 16 entries are put together in LDS (a wave's LDS accesses are carried out in order) and
    // written out once: unused positive slots take the all-ones row, unused negative ones the zeros
    uint32_t *slots = chosen;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    if (lane < 2 + 2 * HALF_BIG_PAIRS) {
        uint32_t v = (lane >= 2 && lane < 2 + 2 * a ? ones_row : zero_row) * row16;
        if (lane == 0) v = (uint32_t)((2 * pairs + 1) | (n > taken ? 0x100 : 0) | (a << 12));
        if (lane == 1) v = (uint32_t)(hv + c % n_types) * row16;
        slots[lane] = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    if (positive) slots[2 + pos_rank] = lit * row16;
    if (negative) slots[2 + 2 * a + neg_rank] = (lit - (uint32_t)hv) * row16;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
    if (lane < 16) rec[lane] = lane == 0 ? slots[0] : slots[lane] << 4;  // rows as byte offsets: nothing to unpack
    // (entries past the 16th follow the include words)
    if (lane >= 16 && lane < 2 + 2 * HALF_BIG_PAIRS) rec[16 + chunks + (lane - 16)] = slots[lane] << 4;
    for (int w = lane; w < chunks; w += 64) {
        uint32_t word = inc[(int64_t)w * B];
        if (w == chunks - 1) word &= filter;
        rec[16 + w] = word;
    }
    if (weights)
        for (int k = lane; k < K; k += 64) wt[(int64_t)c * K + k] = weights[(int64_t)k * C + c];
}

// acc &= the PAIRS row pairs in r, the first A of them positive, the others negated
template <int LW, int PAIRS, int A>
__device__ __forceinline__ void half_combine(LaneWords<LW> &acc, const LaneWords<LW> *r) {
#pragma unroll
    for (int j = 0; j < PAIRS; ++j)
#pragma unroll
        for (int u = 0; u < LW; ++u)
            acc.w[u] = j < A ? acc.w[u] & r[2 * j].w[u] & r[2 * j + 1].w[u] : acc.w[u] & ~(r[2 * j].w[u] | r[2 * j + 1].w[u]);
}

template <int NWAVES, int LW, int LA4, bool LAST, bool FULL>
__global__ __launch_bounds__(NWAVES * 64) void k_tile_two_phase_half(TileLayerArgs a) {
    extern __shared__ uint32_t lds[];
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, C = a.C, K = a.K;
    constexpr int NT = NWAVES * 64;
    constexpr int LA = 4 * LA4;
    const int hv = LA * 16;                      // positive literals = LDS rows 0 .. hv - 1
    const int rows_lds = tg.rows - hv;           // + node types + all ones
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)rows_lds * tw + TILE_LDS_PAD_WORDS);
    // This workgroup's share: a whole tile, or - with a table of segments (tile_segments_part above) - clauses
    // [c_begin, c_end) of a tile whose other clauses other workgroups take.
    int tile_local = blockIdx.x, c_begin = 0, c_end = C;
    if (a.segments) {
        const TileSegment seg = a.segments[blockIdx.x];
        tile_local = seg.tile_local, c_begin = seg.c_begin, c_end = seg.c_end;
        if (c_begin >= c_end) return;  // (an empty share: uniform over the workgroup)
    }
    const bool whole_tile = c_begin == 0 && c_end == C;
    const int tile = a.tile0 + tile_local;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint32_t *bitmap = a.bitmap + (int64_t)tile_local * C * tw;

    {  // the tile's positive rows, then its node-type rows and the all-ones row -> LDS
        const uint4 *src = reinterpret_cast<const uint4 *>(a.tiles + (int64_t)tile * tg.rows * tw);
        uint4 *dst = reinterpret_cast<uint4 *>(bt);
        const int n4 = (rows_lds * tw) >> 2, first4 = (hv * tw) >> 2, skip4 = (hv * tw) >> 2;  // rows hv .. 2 hv - 1 stay out
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
        for (int i = tid; i < TILE_LDS_PAD_WORDS + tg.gpt * K; i += NT) bt[(size_t)rows_lds * tw + i] = 0;
    }
    __syncthreads();

    const bool active = FULL || lane * LW < tw;
    const char *col = reinterpret_cast<const char *>(bt + lane * LW);

    // the graph whose slot this lane's words belong to, and the literal words of the node at the lane's first bit
    const int lpg = tg.lanes_per_graph;
    const int lane_j = lane / lpg;
    const int64_t lane_g = (int64_t)tile * tg.gpt + lane_j;
    const bool has_graph = active && lane_j < tg.gpt && lane_g < a.G;
    // the positive literal words of the node slots of this lane's words (LA / 2 words per slot): the tile's
    // part of `xpos` through a buffer descriptor, so that a load is the descriptor (scalar registers), a
    // 32-bit byte offset per lane and nothing else
    const char *x_base = reinterpret_cast<const char *>(a.xpos) + (int64_t)tile * tw * 32 * (LA * 2);
    const __amdgpu_buffer_rsrc_t x_of_tile =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(x_base), 0, tw * 32 * (LA * 2), BUFFER_RSRC_FLAGS);
    const uint32_t x_lane = (uint32_t)(active ? lane * LW * 32 : 0) * (LA * 2u);
    auto load_x = [&](uint32_t at, uint2 *x) {
        if (LA4 % 2 == 0) {
#pragma unroll
            for (int q = 0; q < LA4; q += 2) {
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(x_of_tile, (int)at + q * 8, 0, 0);
                x[q] = make_uint2(v.x, v.y);
                x[q + 1] = make_uint2(v.z, v.w);
            }
        } else {
#pragma unroll
            for (int q = 0; q < LA4; ++q) {
                const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(x_of_tile, (int)at + q * 8, 0, 0);
                x[q] = make_uint2(v.x, v.y);
            }
        }
    };
    // the clause-major weights, read at a byte offset per lane and a scalar one per clause
    // the include words of a clause (after the 16 entries of its record), the same for every lane, into VECTOR registers
    const __amdgpu_buffer_rsrc_t records =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(a.lists), 0, C * a.stride * 4, BUFFER_RSRC_FLAGS);
    auto load_include = [&](uint32_t record_at) {
        Words<LA> m;
#pragma unroll
        for (int q = 0; q < LA4; ++q) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(records, 64 + 16 * q, (int)record_at, 0);
            m.v[4 * q] = v.x, m.v[4 * q + 1] = v.y, m.v[4 * q + 2] = v.z, m.v[4 * q + 3] = v.w;
        }
        return m;
    };
    const __amdgpu_buffer_rsrc_t weights_of_clauses =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t *>(LAST ? a.wt : nullptr), 0, LAST ? C * K * 4 : 0, BUFFER_RSRC_FLAGS);

    // Votes: lane l belongs to graph j = l / lanes_per_graph of the tile and adds, when a clause holds somewhere in
    // that graph, the clause's weights of the classes i, i + lanes_per_graph, ... (i = l % lanes_per_graph): whether
    // the graph fires is worked out once per lane and clause, and every vote after that is an LDS atomic.  A vote
    // that a lane does not have reads its weight out of the buffer's range, which gives 0 without a memory access,
    // and adds that to a sum of the lane's own: no execution masks to keep.
    const int pairs = tg.gpt * K;
    constexpr int VOTES = 4;
    const int n_votes = (K + lpg - 1) / lpg;
    const bool votes_by_owner = lpg <= 32 && n_votes <= VOTES;
    const bool owner = LAST && votes_by_owner && lane_j < tg.gpt;
    const unsigned long long slot_lanes = lpg >= 64 ? ~0ull : (1ull << lpg) - 1ull;
    const uint32_t graph_lanes = owner ? (uint32_t)slot_lanes : 0u;
    const uint32_t graph_shift = (uint32_t)(owner ? lane_j * lpg : 0);  // first lane of this lane's graph
    uint32_t vote_k_bytes[VOTES], vote_at[VOTES];
#pragma unroll
    for (int v = 0; v < VOTES; ++v) {
        const int i = lane - lane_j * lpg, k = i + lpg * v;
        const bool on = owner && k < K;
        vote_k_bytes[v] = on ? (uint32_t)k * 4u : 0x7FFFFFF0u;
        vote_at[v] = on ? (uint32_t)(lane_j * K + k) : owner && i < K ? (uint32_t)(lane_j * K + i) : 0u;
    }
    const int my_shift = (lane < tg.gpt ? lane : 0) * lpg;

    auto any_bit = [](const LaneWords<LW> &x) {
        uint32_t m = x.w[0];
#pragma unroll
        for (int u = 1; u < LW; ++u) m |= x.w[u];
        return m != 0;
    };
    auto entry_of = [](const Entries16 &rec, int i) { return rec.v[i]; };
    // a positive literal is violated where the node lacks it, a negated one (include words LA / 2 ..)
    // where the node has it: x ? include_neg : include_pos, one 3-input operation per word (the include
    // words are in vector registers, see the loads in the loop below: with two of three operands in
    // scalar registers it is two operations and a move)
    auto violates = [](const Words<LA> &include, const uint2 *x) {
        uint32_t t[2 * LA4];
#pragma unroll
        for (int q = 0; q < LA4; ++q) {
            t[2 * q] = __builtin_amdgcn_bitop3_b32(x[q].x, include.v[2 * q + 2 * LA4], include.v[2 * q], 0xCA);
            t[2 * q + 1] = __builtin_amdgcn_bitop3_b32(x[q].y, include.v[2 * q + 1 + 2 * LA4], include.v[2 * q + 1], 0xCA);
        }
        uint32_t violated = t[0];
#pragma unroll
        for (int w = 1; w < 2 * LA4; ++w) violated |= t[w];
        return violated != 0;
    };
    // the word set with only `bit` set (bit < 32 * LW)
    auto one_hot = [](uint32_t bit) {
        LaneWords<LW> m;
#pragma unroll
        for (int u = 0; u < LW; ++u) m.w[u] = (int)(bit >> 5) == u ? 1u << (bit & 31u) : 0u;
        return m;
    };
    // the word set W without its lowest set bit: W & (W - 1), the decrement carried through the words
    auto without_lowest_bit = [](const LaneWords<LW> &x) {
        LaneWords<LW> r;
        uint32_t borrow = 1u;
#pragma unroll
        for (int u = 0; u < LW; ++u) {
            uint32_t out;
            const uint32_t less = __builtin_subc(x.w[u], 0u, borrow, &out);
            borrow = out;
            r.w[u] = x.w[u] & less;
        }
        return r;
    };

    // Fetching the words of a lane's SECOND surviving slot along with the first's (so that the turns in the open start
    // at the third candidate) paid with 7 row pairs in phase 1 (0.361 -> 0.359 ms per 10,000 graphs); with 8 pairs there
    // are fewer candidates, and its 8 registers are the ones the 16th row needs (with both, the compiler spills).
    constexpr bool SECOND_AHEAD = false;
    struct Pending {
        LaneWords<LW> acc;
        uint2 x[LA4], x2[LA4];   // the words of the lane's first and (for the class sums) second surviving slot
        uint32_t bit;            // the node slot this lane has under test (index into its LW words), ~0 if none
        bool live, test;         // wave-uniform: a clause is pending / its phase 2 runs
        unsigned long long nz;   // lanes with a surviving slot after phase 1
        int weight[VOTES];
        uint32_t weights_at;     // byte offset of the clause's weights
        char *truth_out;
    };

    // Phase 1 and the loads of phase 2.  Every load is issued by all lanes whatever the clause
    // does, so that the number of loads in flight is known when the pending clause is finished.
    auto begin = [&](Pending &p, const Entries16 &rec, const uint2 rec_more, uint32_t weights_at, char *truth_out,
                     const uint32_t *record_next, Entries16 &next, uint2 &next_more) {
        p.live = true;
        p.weights_at = weights_at;
        p.truth_out = truth_out;
        if (LAST) {  // needed only if the clause fires
#pragma unroll
            for (int v = 0; v < VOTES; ++v)
                p.weight[v] = (int)__builtin_amdgcn_raw_buffer_load_b32(weights_of_clauses, (int)vote_k_bytes[v], (int)weights_at, 0);
        }
        const uint32_t header = rec.v[0] & 0xFFFFu;
        const uint32_t positive_pairs = header >> 12;
        LaneWords<LW> acc, r[2 * HALF_BIG_PAIRS];
        acc.load(col + entry_of(rec, 1));  // the node-type row: zero past the graphs' nodes and in unused lanes
        if (!FULL && !active)
#pragma unroll
            for (int u = 0; u < LW; ++u) acc.w[u] = 0u;
        if ((header & 0xFFu) > 7u) {
#pragma unroll
            for (int i = 0; i < 2 * HALF_BIG_PAIRS; ++i)
                r[i].load(col + (i + 2 < 16 ? entry_of(rec, i + 2 < 16 ? i + 2 : 0) : i + 2 == 16 ? rec_more.x : rec_more.y));
            switch (positive_pairs) {
                case 0: half_combine<LW, HALF_BIG_PAIRS, 0>(acc, r); break;
                case 1: half_combine<LW, HALF_BIG_PAIRS, 1>(acc, r); break;
                case 2: half_combine<LW, HALF_BIG_PAIRS, 2>(acc, r); break;
                case 3: half_combine<LW, HALF_BIG_PAIRS, 3>(acc, r); break;
                case 4: half_combine<LW, HALF_BIG_PAIRS, 4>(acc, r); break;
                case 5: half_combine<LW, HALF_BIG_PAIRS, 5>(acc, r); break;
                case 6: half_combine<LW, HALF_BIG_PAIRS, 6>(acc, r); break;
                case 7: half_combine<LW, HALF_BIG_PAIRS, 7>(acc, r); break;
                default: half_combine<LW, HALF_BIG_PAIRS, HALF_BIG_PAIRS>(acc, r); break;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 6; ++i) r[i].load(col + entry_of(rec, i + 2));
            switch (positive_pairs) {
                case 0: half_combine<LW, 3, 0>(acc, r); break;
                case 1: half_combine<LW, 3, 1>(acc, r); break;
                case 2: half_combine<LW, 3, 2>(acc, r); break;
                default: half_combine<LW, 3, 3>(acc, r); break;
            }
        }
        // (the next record is requested only now: scalar loads and LDS reads are waited for with one counter, so a
        // request before the rows would have been waited for along with them)
        next = *reinterpret_cast<const Entries16 *>(record_next);
        next_more = *reinterpret_cast<const uint2 *>(record_next + 16 + LA);
        // lowest surviving slot of the lane: the smallest of its words' lowest set bits (~0 for a word without
        // one, which survives the OR with the word's base and loses every comparison: no slot)
        uint32_t bit = lowest_bit_or_ones(acc.w[0]);
#pragma unroll
        for (int u = 1; u < LW; ++u) {
            const uint32_t here = lowest_bit_or_ones(acc.w[u]) | (uint32_t)u * 32u;
            bit = here < bit ? here : bit;
        }
        // (no slot survives in lanes without a graph: the node-type row is zero there)
        p.nz = __ballot(bit != ~0u);
        p.test = (header & 0x100u) && p.nz != 0;
        p.bit = bit;
        // lanes with nothing to test all read the tile's first slot (one cache line for the wave)
        load_x(bit != ~0u ? x_lane + bit * (LA * 2u) : 0u, p.x);
        if (LAST && SECOND_AHEAD) {
            // The second surviving slot's words come along: a first candidate fails often enough, and a test that
            // starts only then has its memory round trip in the open.
            const LaneWords<LW> after = without_lowest_bit(acc);
            uint32_t bit2 = lowest_bit_or_ones(after.w[0]);
#pragma unroll
            for (int u = 1; u < LW; ++u) {
                const uint32_t here = lowest_bit_or_ones(after.w[u]) | (uint32_t)u * 32u;
                bit2 = here < bit2 ? here : bit2;
            }
            load_x(bit2 != ~0u ? x_lane + bit2 * (LA * 2u) : 0u, p.x2);
        }
        p.acc = acc;
    };

    // The rest of phase 2, then the clause's votes (or its truth row).
    auto finish = [&](Pending &p, const Words<LA> &include) {
        if (!p.live) return;
        p.live = false;
        LaneWords<LW> acc = p.acc;
        unsigned long long nz = p.nz;
        bool settled = false;
        if (LAST && p.test) {
            // Class sums only ask whether the clause is true at SOME node of a graph
            // (kernels.py:297-308): a lane whose first candidate holds has settled that for its graph.
            // Only a lane whose first candidate failed and that has others needs more tests (rare: then
            // the exact path below runs).
            const bool tested = p.bit != ~0u;
            int slots_left = 0;
#pragma unroll
            for (int u = 0; u < LW; ++u) slots_left += __popc(acc.w[u]);
            bool holds = tested && (!violates(include, p.x) || (SECOND_AHEAD && slots_left > 1 && !violates(include, p.x2)));
            const bool more = tested && !holds && slots_left > (SECOND_AHEAD ? 2 : 1);
            if (__ballot(more) == 0ull) {
                nz = __ballot(holds);
                settled = true;
            } else {
                // Both candidates of some lane failed and it has others.  All such lanes test their next candidate
                // at the same time, one memory round trip per turn, and a lane stops at its first candidate that
                // holds: as many turns as the unluckiest lane needs.  (With many candidates left somewhere the
                // rows of all the clause's literals are ANDed instead, below.)
                // (the candidate under test is always the lowest set bit of the lane's words taken as one number W:
                // W & (W - 1) takes it out)
                LaneWords<LW> rest = SECOND_AHEAD ? without_lowest_bit(without_lowest_bit(acc)) : without_lowest_bit(acc);
                int others = 0;
#pragma unroll
                for (int u = 0; u < LW; ++u) {
                    rest.w[u] = more ? rest.w[u] : 0u;
                    others += __popc(rest.w[u]);
                }
                if (__ballot(others + (SECOND_AHEAD ? 1 : 0) >= TWO_PHASE_WALK_FROM) == 0ull) {
                    while (__ballot(any_bit(rest)) != 0ull) {
                        uint32_t bit = lowest_bit_or_ones(rest.w[0]);
#pragma unroll
                        for (int u = 1; u < LW; ++u) {
                            const uint32_t here = lowest_bit_or_ones(rest.w[u]) | (uint32_t)u * 32u;
                            bit = here < bit ? here : bit;
                        }
                        const bool searching = bit != ~0u;
                        uint2 x[LA4];
                        load_x(searching ? x_lane + bit * (LA * 2u) : 0u, x);
                        const LaneWords<LW> next = without_lowest_bit(rest);
                        const bool ok = searching && !violates(include, x);
                        holds = holds || ok;
#pragma unroll
                        for (int u = 0; u < LW; ++u) rest.w[u] = ok ? 0u : next.w[u];
                    }
                    nz = __ballot(holds);
                    settled = true;
                }
            }
        }
        if (p.test && !settled) {
            const bool tested = p.bit != ~0u;
            const bool failed = violates(include, p.x) && tested;
            // the lane's other surviving slots
            const LaneWords<LW> hot = one_hot(p.bit);
            LaneWords<LW> rest;
#pragma unroll
            for (int u = 0; u < LW; ++u) {
                rest.w[u] = tested ? acc.w[u] & ~hot.w[u] : 0u;
                acc.w[u] = failed ? rest.w[u] : acc.w[u];
            }
            if (__ballot(any_bit(rest)) != 0) {
                int others = 0;
#pragma unroll
                for (int u = 0; u < LW; ++u) others += __popc(rest.w[u]);
                if (__builtin_expect(__ballot(others >= TWO_PHASE_WALK_FROM) != 0, 0)) {
                    // Phase 1 has left some lane several slots (its literals hold nearly everywhere), and
                    // testing them costs a memory round trip each.  The rows of ALL the clause's literals are
                    // ANDed instead (row l is literal l's; a negated literal l + hv takes the complement of
                    // row l; unused reads take the all-ones row, resp. the zeroed words after the rows).
                    acc = p.acc;
                    const uint32_t row_bytes = (uint32_t)tw * 4u;
                    const uint32_t ones = (uint32_t)(rows_lds - 1), zeros = (uint32_t)rows_lds;
                    uint32_t include_of_lane = 0u;  // lane w holds include word w: one copy of the loop below
#pragma unroll
                    for (int w = 0; w < LA; ++w) include_of_lane = lane == w ? include.v[w] : include_of_lane;
#pragma unroll 1
                    for (int w = 0; w < LA; ++w) {
                        uint32_t m = __builtin_amdgcn_readlane(include_of_lane, w);
                        const bool negated = w >= LA / 2;
                        const uint32_t first = (uint32_t)((negated ? w - LA / 2 : w) * 32), unused = negated ? zeros : ones;
                        while (m) {
                            LaneWords<LW> r[8];
#pragma unroll
                            for (int u = 0; u < 8; ++u) {
                                const uint32_t row = m ? first + (uint32_t)__builtin_ctz(m) : unused;
                                m &= m - 1u;
                                r[u].load(col + row * row_bytes);
                            }
                            if (negated) {
#pragma unroll
                                for (int u = 0; u < 8; ++u)
#pragma unroll
                                    for (int v = 0; v < LW; ++v) acc.w[v] &= ~r[u].w[v];
                            } else {
#pragma unroll
                                for (int u = 0; u < 8; ++u)
#pragma unroll
                                    for (int v = 0; v < LW; ++v) acc.w[v] &= r[u].w[v];
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < LW; ++u) {
                        uint32_t todo = rest.w[u];
                        while (todo) {
                            const int b = __ffs(todo) - 1;
                            todo &= todo - 1;
                            uint2 x[LA4];
                            load_x(x_lane + (uint32_t)(u * 32 + b) * (LA * 2u), x);
                            if (violates(include, x)) acc.w[u] &= ~(1u << b);
                        }
                    }
                }
            }
            nz = __ballot(any_bit(acc));
        }
        if (!LAST) {
            if (active) acc.store(p.truth_out);
            return;
        }
        if (nz == 0) return;
        // graph j owns lanes [j * lanes_per_graph, (j + 1) * lanes_per_graph)
        if (votes_by_owner) {
            if (((uint32_t)(nz >> graph_shift) & graph_lanes) != 0) {
#pragma unroll
                for (int v = 0; v < VOTES; ++v)
                    if (v < n_votes) atomicAdd(&sums[vote_at[v]], p.weight[v]);
            }
        } else {
            const unsigned long long gm = __ballot(lane < tg.gpt && ((nz >> my_shift) & slot_lanes) != 0);
            const int32_t *weights = a.wt + (p.weights_at >> 2);
            for (int q = lane; q < pairs; q += 64) {
                const int j = q / K, k = q - j * K;
                if ((gm >> j) & 1ull) atomicAdd(&sums[q], weights[k]);
            }
        }
    };

    // Clause records: the 16 words of row entries are fetched one clause ahead of phase 1 (scalar
    // loads), the include words when the clause's phase 1 is over, just before the other clause's
    // (vector loads: they are first needed when the clause is finished, one phase 1 later).  Pointers
    // and offsets step by NWAVES clauses; past the end they stay on the wave's last clause (a valid
    // address whose data is not used).
    const int64_t rec_step = (int64_t)NWAVES * a.stride;
    const uint32_t wt_step = (uint32_t)(NWAVES * K) * 4u;
    const int64_t truth_step = (int64_t)NWAVES * tw * 4;
    const int first = c_begin + wave < c_end ? c_begin + wave : c_begin;
    const uint32_t *rec_a = a.lists + (int64_t)first * a.stride;
    const uint32_t at_step = (uint32_t)(NWAVES * a.stride) * 4u;
    uint32_t at_a = (uint32_t)(first * a.stride) * 4u;  // rec_a as a byte offset
    uint32_t wt_a = LAST ? (uint32_t)(first * K) * 4u : 0u;
    char *truth_a = reinterpret_cast<char *>(bitmap + (int64_t)first * tw + (active ? lane * LW : 0));
    Entries16 ea = *reinterpret_cast<const Entries16 *>(rec_a);
    uint2 ea_more = *reinterpret_cast<const uint2 *>(rec_a + 16 + LA), eb_more;
    Pending pa, pb;
    pa.live = pb.live = false;
    uint32_t at_pending = at_a;  // the record of the clause in pb (a valid record while there is none)
    for (int c = c_begin + wave; c < c_end; c += 2 * NWAVES) {
        const bool has_b = c + NWAVES < c_end;
        const uint32_t *rec_b = has_b ? rec_a + rec_step : rec_a;
        const uint32_t wt_b = LAST && has_b ? wt_a + wt_step : wt_a;
        const uint32_t at_b = has_b ? at_a + at_step : at_a;
        char *truth_b = has_b ? truth_a + truth_step : truth_a;
        // The include words of the pending clause are requested before the phase 1 that runs ahead of its end,
        // so only one clause's are in registers at a time.
        Words<LA> include = load_include(at_pending);
        Entries16 eb;
        begin(pa, ea, ea_more, wt_a, truth_a, rec_b, eb, eb_more);
        finish(pb, include);
        include = load_include(at_a);
        const bool has_a = c + 2 * NWAVES < c_end;
        rec_a = has_a ? rec_b + rec_step : rec_b;
        const uint32_t wt_next = LAST && has_a ? wt_b + wt_step : wt_b;
        at_a = has_a ? at_b + at_step : at_b;
        char *truth_next = has_a ? truth_b + truth_step : truth_b;
        // without a second clause this repeats the first one and drops the result: keeping the
        // sequence of loads the same on every trip lets the waits stay partial
        begin(pb, eb, eb_more, wt_b, truth_b, rec_a, ea, ea_more);
        pb.live = has_b;
        finish(pa, include);
        wt_a = wt_next;
        truth_a = truth_next;
        at_pending = at_b;
    }
    if (pb.live) finish(pb, load_include(at_pending));
    if (!LAST) return;
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NT) {
        int64_t g = g0 + i / K;
        if (g >= a.first_graph && g < (int64_t)a.first_graph + a.n_graphs) {
            int32_t *out = &a.class_sum[(g - a.first_graph) * K + (i % K)];
            if (whole_tile)
                *out = sums[i];
            else if (sums[i] != 0)
                atomicAdd(out, sums[i]);  // a tile shared with other workgroups (tile_segments_part cleared its sums)
        }
    }
}

// ---------------------------------------------------------------------------
// The two-phase layer 0 for nodes with many literal words (any LA), tiles of
// whole-word slots whose rows are staged in LDS or read in place.  Phase 1 as
// above; in phase 2 the surviving node slots are walked on the scalar unit, 8 at
// a time, and for each one lane w compares include word w with the node's
// literal word w (one coalesced load per node and 64 words).  With the rows
// read in place nothing ties a tile to one workgroup, so several workgroups
// share a tile's clauses (truth rows only: the votes of LAST need one
// workgroup per tile).
template <int NWAVES, int LW, int SRC, bool LAST>
__global__ __launch_bounds__(NWAVES * 64) void k_tile_two_phase_wide(TileLayerArgs a, int LA, int n_tiles, int splits,
                                                                      int pack) {
    extern __shared__ uint32_t lds[];
    // Workgroups go to the 8 XCDs in turn, and each XCD has its own L2: the workgroups that share a
    // tile (its rows are read in place, again and again) are given to one XCD, one after the other,
    // so that the few tiles an XCD works on at a time stay in its L2.  1-D grid of
    // ceil(groups / 8) * 8 * splits workgroups, a group being `pack` consecutive tiles: a narrow tile
    // (rows of at most 32 words, rows read in place, truth rows only) leaves half of a wave's lanes or more
    // without a word, so a wave takes 64 / tw tiles at once, lane l on word l % tw of tile l / tw of the
    // group - the clause's row offsets are the same for every tile, and everything else is per lane.
    const int xcd = blockIdx.x & 7, turn = blockIdx.x >> 3;
    const int split = turn % splits, group_of_launch = (turn / splits) * 8 + xcd;
    const int tile_of_launch = group_of_launch * pack;  // the group's first tile
    if (tile_of_launch >= n_tiles) return;
    const TileGeom &tg = a.tg;
    const int tw = tg.tw, C = a.C, K = a.K;
    constexpr int NT = NWAVES * 64;
    const int n_rows_lds = SRC == ROWS_STAGED ? tg.rows : 0;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)n_rows_lds * tw + TILE_LDS_PAD_WORDS);
    uint32_t *first_node = (uint32_t *)(sums + tg.gpt * K);  // [pack][gpt] row of X of each graph's node 0
    uint32_t *node_count = first_node + pack * tg.gpt;       // [pack][gpt]
    const int tile = a.tile0 + tile_of_launch;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this lane's tile of the group and its first word there
    const int sub = pack > 1 ? lane / tw : 0, word_of_lane = pack > 1 ? lane - sub * tw : lane * LW;
    const bool tile_exists = sub < pack && tile_of_launch + sub < n_tiles;  // (the last lanes may be left over)
    uint32_t *bitmap = a.bitmap + (int64_t)(tile_of_launch + (tile_exists ? sub : 0)) * C * tw;

    if (SRC == ROWS_STAGED) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.tiles + (int64_t)tile * tg.rows * tw);
        uint4 *dst = reinterpret_cast<uint4 *>(bt);
        const int n4 = (tg.rows * tw) >> 2;
        for (int i = tid; i < n4; i += NT) dst[i] = src[i];
    }
    for (int i = tid; i < TILE_LDS_PAD_WORDS + tg.gpt * K; i += NT) bt[(size_t)n_rows_lds * tw + i] = 0;
    for (int j = tid; j < pack * tg.gpt; j += NT) {
        const int64_t g = (int64_t)tile * tg.gpt + j;  // (the tiles of a group follow each other: so do their graphs)
        first_node[j] = g < a.G ? a.node_index[g] : 0u;
        node_count[j] = g < a.G ? a.n_nodes[g] : 0u;
    }
    __syncthreads();

    const bool active = pack > 1 ? tile_exists : lane * LW < tw;
    const char *col = SRC == ROWS_GLOBAL
                          ? reinterpret_cast<const char *>(a.tiles + (int64_t)(tile + (active ? sub : 0)) * tg.rows * tw +
                                                           (active ? word_of_lane : 0))
                          : reinterpret_cast<const char *>(bt + lane * LW);
    const int pairs = tg.gpt * K;
    const int my_shift = (lane < tg.gpt ? lane : 0) * tg.lanes_per_graph;
    const unsigned long long slot_lanes = tg.lanes_per_graph >= 64 ? ~0ull : (1ull << tg.lanes_per_graph) - 1ull;

    auto any_bit = [](const LaneWords<LW> &x) {
        uint32_t m = x.w[0];
#pragma unroll
        for (int u = 1; u < LW; ++u) m |= x.w[u];
        return m != 0;
    };
    auto entry_of = [](const Packed8 &rec, int i) { return ((rec.v[i >> 1] >> ((i & 1) * 16)) & 0xFFFFu) << 4; };

    // Per word of this lane: where in X the literal words of the node at the word's bit 0 are, and whether the
    // word belongs to a graph with nodes (a graph without nodes keeps its bit 0 untested).  Phase 2 hands
    // these round with readlane instead of dividing and looking the graph up for every word it visits.
    uint32_t x_lo[LW], x_hi[LW], testable[LW];
#pragma unroll
    for (int u = 0; u < LW; ++u) {
        const int tile_word = word_of_lane + u;
        const int gj = tg.slot_words > 0 ? tile_word / tg.slot_words : 0;
        const bool owned = tg.slot_words > 0 && gj < tg.gpt && active;
        const int node0 = owned ? (tile_word - gj * tg.slot_words) * 32 : 0;
        const int graph_of_group = sub * tg.gpt + gj;
        const uint64_t at = (uint64_t)(((int64_t)(owned ? first_node[graph_of_group] : 0u) + node0) * LA);  // in words from X
        x_lo[u] = (uint32_t)at, x_hi[u] = (uint32_t)(at >> 32);
        testable[u] = owned && node_count[graph_of_group] != 0u ? 0xFFFFFFFFu : 0u;
    }

    const int c_step = NWAVES * splits;
    const int c_first = wave + NWAVES * split;
    const int valid = c_first < C ? c_first : 0;
    struct Rows {
        LaneWords<LW> r[15];
    };
    // phase 1, first half: the reads of the clause's 7 or 15 rows are sent off
    auto issue = [&](const Packed8 &rec, Rows &rows) {
        if ((rec.v[0] & 0xFFu) > 7u) {
#pragma unroll
            for (int i = 0; i < 15; ++i) rows.r[i].load(col + entry_of(rec, i + 1));
        } else {
#pragma unroll
            for (int i = 0; i < 7; ++i) rows.r[i].load(col + entry_of(rec, i + 1));
        }
    };
    // the rest of the clause
    auto finish = [&](int c, const Packed8 &rec, const uint32_t *record, uint32_t include0, const Rows &rows) {
        const uint32_t header = rec.v[0] & 0xFFFFu;
        LaneWords<LW> acc;
#pragma unroll
        for (int u = 0; u < LW; ++u) acc.w[u] = active ? 0xFFFFFFFFu : 0u;
        if ((header & 0xFFu) > 7u) {
#pragma unroll
            for (int i = 0; i < 15; ++i)
#pragma unroll
                for (int u = 0; u < LW; ++u) acc.w[u] &= rows.r[i].w[u];
        } else {
#pragma unroll
            for (int i = 0; i < 7; ++i)
#pragma unroll
                for (int u = 0; u < LW; ++u) acc.w[u] &= rows.r[i].w[u];
        }
        unsigned long long nz = __ballot(any_bit(acc));
        // Phase 2 costs a memory round trip per 8 surviving slots, ANDing the rows of all the clause's
        // literals one per 8 literals: when more than twice as many slots survive as the clause has literals
        // (its rarest literals hold nearly everywhere: negated ones, mostly), the rows are walked instead,
        // as k_tile_layer does (row l belongs to literal l; unused reads take the all-ones row).  (Measured on
        // the colour workload, 2,000 graphs: the kernel takes 11.2 ms with one slot per literal as the limit,
        // 10.1 ms with two, 10.5 with four, 11.7 never walking, 13.8 with half a slot.)
        bool walk = false;
        if ((header & 0x100u) && nz != 0) {
            int survivors = 0, literals = __popc(include0);
#pragma unroll
            for (int u = 0; u < LW; ++u) survivors += __popc(acc.w[u]);
            for (int w0 = 64; w0 < LA; w0 += 64) literals += w0 + lane < LA ? __popc(record[8 + w0 + lane]) : 0;
            for (int off = 32; off > 0; off >>= 1) {
                survivors += __shfl_xor(survivors, off);
                literals += __shfl_xor(literals, off);
            }
            walk = survivors > literals * a.walk_factor;
        }
        if (walk) {
            const uint32_t row_bytes = (uint32_t)tw * 4u, ones = (uint32_t)(tg.rows - 1);
            for (int w0 = 0; w0 < LA; w0 += 64) {
                const uint32_t include = w0 == 0 ? include0 : (w0 + lane < LA ? record[8 + w0 + lane] : 0u);
                unsigned long long has = __ballot(include != 0u);
                while (has) {
                    const int L = __ffsll((long long)has) - 1;
                    has &= has - 1;
                    uint32_t m = __builtin_amdgcn_readlane(include, L);
                    const uint32_t base = (uint32_t)(w0 + L) * 32u;
                    while (m) {
                        LaneWords<LW> r[8];
#pragma unroll
                        for (int q = 0; q < 8; ++q) {
                            const uint32_t lit = m ? base + (uint32_t)__builtin_ctz(m) : ones;
                            m &= m - 1u;
                            r[q].load(col + (size_t)lit * row_bytes);
                        }
#pragma unroll
                        for (int q = 0; q < 8; ++q)
#pragma unroll
                            for (int u = 0; u < LW; ++u) acc.w[u] &= r[q].w[u];
                    }
                }
            }
            nz = __ballot(any_bit(acc));
        } else if ((header & 0x100u) && nz != 0) {
            // Phase 2: the surviving slots, wherever in the wave they sit, are taken 8 at a time (one
            // memory round trip per 8): a cursor on the scalar unit walks the lanes that hold some, the
            // words of such a lane and the bits of such a word.
            for (int w0 = 0; w0 < LA; w0 += 64) {
                const bool in_row = w0 + lane < LA;
                const uint32_t include = w0 == 0 ? include0 : (in_row ? record[8 + w0 + lane] : 0u);
                unsigned long long live = __ballot(any_bit(acc));
                int at_lane = 0, at_word = LW, next_word = LW;
                uint32_t bits = 0u;
                const uint32_t *x_of_word = a.X;  // literal words w0 + lane of the node at bit 0 of the cursor's word
                // the next surviving slot as lane | word << 8 | bit << 16, or -1
                auto next_slot = [&]() {
                    while (bits == 0u) {
                        if (next_word >= LW) {
                            if (live == 0ull) return -1;
                            at_lane = __ffsll((long long)live) - 1;
                            live &= live - 1;
                            next_word = 0;
                        }
                        uint32_t word = 0u, lo = 0u, hi = 0u;
#pragma unroll
                        for (int u = 0; u < LW; ++u)
                            if (u == next_word) {
                                word = __builtin_amdgcn_readlane(acc.w[u] & testable[u], at_lane);
                                lo = __builtin_amdgcn_readlane(x_lo[u], at_lane);
                                hi = __builtin_amdgcn_readlane(x_hi[u], at_lane);
                            }
                        at_word = next_word++;
                        x_of_word = a.X + (int64_t)(((uint64_t)hi << 32) | lo) + w0 + (in_row ? lane : 0);
                        bits = word;
                    }
                    const int b = __builtin_ctz(bits);
                    bits &= bits - 1u;
                    return at_lane | at_word << 8 | b << 16;
                };
                for (;;) {
                    int slot[8];
                    uint32_t xs[8];
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        slot[q] = next_slot();
                        const uint32_t *x = slot[q] >= 0 ? x_of_word + (int64_t)(slot[q] >> 16) * LA : a.X;
                        xs[q] = *x;
                    }
                    if (slot[0] < 0) break;
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        if (slot[q] < 0) continue;
                        if (__ballot((include & ~xs[q]) != 0u) == 0ull) continue;
                        const uint32_t keep = ~(1u << (slot[q] >> 16));
#pragma unroll
                        for (int u = 0; u < LW; ++u)
                            if (lane == (slot[q] & 0xFF) && u == ((slot[q] >> 8) & 0xFF)) acc.w[u] &= keep;
                    }
                    if (slot[7] < 0) break;
                }
            }
            nz = __ballot(any_bit(acc));
        }
        if (!LAST) {
            if (active) acc.store(reinterpret_cast<char *>(bitmap + (int64_t)c * tw + word_of_lane));
            return;
        }
        if (nz == 0) return;
        const int32_t *weights_of_clause = a.wt + (int64_t)c * K;
        const unsigned long long gm = __ballot(lane < tg.gpt && ((nz >> my_shift) & slot_lanes) != 0);
        for (int p = lane; p < pairs; p += 64) {
            int j = p / K, k = p - j * K;
            if ((gm >> j) & 1ull) atomicAdd(&sums[p], weights_of_clause[k]);
        }
        };
    // Two clauses of a wave are under way at a time: the rows of both are requested before either is
    // ANDed (rows read in place come from L2 or further: a clause is a chain of memory round trips).
    // Without a second clause the first is repeated and the result dropped.
    const int64_t pair_step = 2 * (int64_t)c_step;
    Packed8 next_a = *reinterpret_cast<const Packed8 *>(a.lists + (int64_t)valid * a.stride);
    Packed8 next_b = *reinterpret_cast<const Packed8 *>(a.lists + (int64_t)(c_first + c_step < C ? c_first + c_step : valid) * a.stride);
    for (int c = c_first; c < C; c += 2 * c_step) {
        const bool has_b = c + c_step < C;
        const int cb = has_b ? c + c_step : c;
        const uint32_t *record_a = a.lists + (int64_t)c * a.stride, *record_b = a.lists + (int64_t)cb * a.stride;
        const Packed8 rec_a = next_a, rec_b = next_b;
        const int64_t na = c + pair_step < C ? c + pair_step : valid, nb = c + pair_step + c_step < C ? c + pair_step + c_step : na;
        next_a = *reinterpret_cast<const Packed8 *>(a.lists + na * a.stride);
        next_b = *reinterpret_cast<const Packed8 *>(a.lists + nb * a.stride);
        // the first 64 include words travel with the rows (phase 2 would otherwise wait for them alone)
        const uint32_t include0_a = lane < LA ? record_a[8 + lane] : 0u;
        const uint32_t include0_b = lane < LA ? record_b[8 + lane] : 0u;
        Rows rows_a, rows_b;
        issue(rec_a, rows_a);
        issue(rec_b, rows_b);
        finish(c, rec_a, record_a, include0_a, rows_a);
        if (has_b) finish(cb, rec_b, record_b, include0_b, rows_b);
    }
    if (!LAST) return;
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NT) {
        int64_t g = g0 + i / K;
        if (g >= a.first_graph && g < (int64_t)a.first_graph + a.n_graphs)
            a.class_sum[(g - a.first_graph) * K + (i % K)] = sums[i];
    }
}
