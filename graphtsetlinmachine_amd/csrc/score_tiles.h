// Batched depth-1 inference on literal-major tiles.
//
// The dense form of clause evaluation tests every clause against every word
// of every node (CLAUSES x nodes x LA_CHUNKS word operations per graph) and is
// bound by integer VALU throughput, not by HBM.  A clause is an AND of few
// literals, so this path turns the data instead: for a tile of graphs it keeps
// one bit-row per LITERAL (bit n of the row = that literal at node slot n of
// the tile), staged in LDS, and a clause's truth over all node slots of the
// tile is the AND of the rows of its included literals only.  The result is
// the same bits as kernels.py:443-466 computes; no clause/node bitmap is
// written because `evaluate` (kernels.py:297-315) only needs "true at some
// node of the graph".
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

struct TileGeom {
    int slot_bits;        // bits per graph slot
    int slot_words;       // words per graph slot (0 when slot_bits < 32)
    int gpt;              // graphs per tile
    int tw;               // words per tile row
    int rows;             // LITERALS + node types + 1
    int n_tiles;
    int lw;               // words of a row held by one lane (1, 2 or 4)
    int lanes_per_graph;  // slot_words / lw (0 when slot_bits < 32)
    int ok;               // geometry supported by the fused kernel
};

constexpr size_t TILE_LDS_BUDGET = 156 * 1024;  // of the 160 KB per CU
constexpr int TILE_LDS_PAD_WORDS = 256;         // readable words after the last row

inline size_t tile_lds_bytes(const TileGeom &g, int classes) {
    return ((size_t)g.rows * g.tw + TILE_LDS_PAD_WORDS + (size_t)g.gpt * classes) * 4;
}

// The widest lanes (most graphs per wave instruction) whose tile fits in LDS.
inline TileGeom tile_geometry(int literals, int n_types, int max_nodes, int n_graphs, int classes, int max_lw = 4) {
    TileGeom last{};
    if (max_nodes < 1) max_nodes = 1;
    for (int lw = max_lw; lw >= 1; lw >>= 1) {
        TileGeom g{};
        g.lw = lw;
        const int max_words = 64 * lw;
        g.rows = literals + n_types + 1;
        if (max_nodes <= 16) {
            int s = 1;
            while (s < max_nodes) s <<= 1;
            g.slot_bits = s;
            // many literals: narrower rows (fewer graphs per tile) until the tile fits in LDS
            g.tw = max_words;
            g.gpt = g.tw * 32 / s;
            while (g.tw > 4 * lw && tile_lds_bytes(g, classes) > TILE_LDS_BUDGET) {
                g.tw >>= 1;
                g.gpt = g.tw * 32 / s;
            }
        } else {
            g.slot_words = ((max_nodes - 1) / 32 + 1 + lw - 1) / lw * lw;
            g.slot_bits = g.slot_words * 32;
            g.lanes_per_graph = g.slot_words / lw;
            g.gpt = g.slot_words <= max_words ? max_words / g.slot_words : 0;
            g.tw = g.gpt * g.slot_words;
            if (g.tw & 3) g.tw = (g.tw + 3) & ~3;  // rows stay 16-byte aligned
        }
        g.rows = literals + n_types + 1;
        g.n_tiles = g.gpt > 0 ? (n_graphs + g.gpt - 1) / g.gpt : 0;
        g.ok = g.gpt > 0 && tile_lds_bytes(g, classes) <= TILE_LDS_BUDGET;
        if (g.ok) return g;
        last = g;
    }
    last.ok = 0;
    return last;
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
// LDS byte offsets (row * tw * 4).  Entry 0 = number of 8-entry blocks in use,
// entry 1 = the row of the clause's node type (kernels.py:447), then its
// included literals in `order`: the ones that hold least often come first, so
// the running AND dies (and the walk stops) as early as it can; the order does
// not change the result.  The list starts with a chunk of 32 entries that the
// scoring kernel fetches one clause ahead; unused entries point at the
// all-ones row.  Also the weights clause-major.
__global__ void k_compile_clauses(const uint32_t *__restrict__ bank, int C, int LA, int B, uint32_t filter, int K,
                                  const int32_t *__restrict__ weights, int literals, int n_types, int tw,
                                  int stride, const uint32_t *__restrict__ order, uint32_t *__restrict__ lists,
                                  int32_t *__restrict__ wt) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (c >= C) return;
    const uint32_t row_bytes = (uint32_t)tw * 4u;
    const uint32_t ones = (uint32_t)(literals + n_types) * row_bytes;
    uint32_t *list = lists + (int64_t)c * stride;
    const uint32_t *inc = bank + (int64_t)c * LA * B + (B - 1);
    if (lane == 0) list[1] = (uint32_t)(literals + c % n_types) * row_bytes;
    int n = 2;
    for (int r0 = 0; r0 < literals; r0 += 64) {
        int r = r0 + lane;
        uint32_t lit = r < literals ? order[r] : 0u;
        uint32_t w = lit >> 5;
        uint32_t word = inc[(int64_t)w * B];
        if ((int)w == LA - 1) word &= filter;
        bool included = r < literals && ((word >> (lit & 31)) & 1u);
        unsigned long long mask = __ballot(included);
        if (included) list[n + __popcll(mask & ((1ull << lane) - 1ull))] = lit * row_bytes;
        n += __popcll(mask);
    }
    const int padded = (n + 7) & ~7;
    const int fill_to = padded < 32 ? 32 : (padded + 15) & ~15;
    for (int i = n + lane; i < fill_to; i += 64) list[i] = ones;
    if (lane == 0) list[0] = (uint32_t)(padded >> 3);
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
};
template <>
struct LaneWords<2> {
    uint32_t w[2];
    __device__ __forceinline__ void load(const char *p) {
        uint2 v = *reinterpret_cast<const uint2 *>(p);
        w[0] = v.x;
        w[1] = v.y;
    }
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
};

// One workgroup per tile.  The tile's bit-rows are copied to LDS once; each
// wave then walks its share of the clauses.  The clause id and its row list
// are wave-uniform: the first 32 entries of a clause arrive by scalar loads
// issued while the previous clause is being evaluated.  Lane L holds words
// [L*LW, (L+1)*LW) of the running AND.
template <int NWAVES, int LW>
__global__ __launch_bounds__(NWAVES * 64) void k_score_tiles(
    const uint32_t *__restrict__ tiles, TileGeom tg, int C, int K, const uint32_t *__restrict__ lists, int stride,
    const int32_t *__restrict__ wt, int tile0, int first_graph, int n_graphs, int32_t *__restrict__ class_sum) {
    extern __shared__ uint32_t lds[];
    const int tw = tg.tw;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)tg.rows * tw + TILE_LDS_PAD_WORDS);
    const int tile = tile0 + blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    {  // tile -> LDS, 16 bytes per thread and trip, several loads in flight
        const uint4 *src = reinterpret_cast<const uint4 *>(tiles + (int64_t)tile * tg.rows * tw);
        uint4 *dst = reinterpret_cast<uint4 *>(bt);
        const int n4 = (tg.rows * tw) >> 2;  // tw is a multiple of 4
        for (int i = tid; i < n4; i += NWAVES * 64 * 4) {
            uint4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int at = i + u * NWAVES * 64;
                v[u] = at < n4 ? src[at] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int at = i + u * NWAVES * 64;
                if (at < n4) dst[at] = v[u];
            }
        }
        for (int i = tid; i < TILE_LDS_PAD_WORDS + tg.gpt * K; i += NWAVES * 64) bt[tg.rows * tw + i] = 0;
    }
    __syncthreads();

    // Lanes past the row width read the words after the row (inside the
    // allocation) so that they fall on banks no other lane of the access uses;
    // their running AND starts at 0 and stays 0.
    const bool active = lane * LW < tw;
    const char *col = reinterpret_cast<const char *>(bt + lane * LW);

    // lane p < gpt*K adds weight k = p % K to graph j = p / K of the tile
    const int pairs = tg.gpt * K;
    const int my_j = lane / K, my_k = lane - my_j * K;
    const bool pair_lane = tg.slot_words > 0 && lane < pairs;
    const int my_shift = (lane < tg.gpt ? lane : 0) * tg.lanes_per_graph;
    const unsigned long long slot_lanes = tg.lanes_per_graph >= 64 ? ~0ull : (1ull << tg.lanes_per_graph) - 1ull;

    auto any_bit = [](const LaneWords<LW> &a) {
        uint32_t m = a.w[0];
#pragma unroll
        for (int u = 1; u < LW; ++u) m |= a.w[u];
        return m != 0;
    };
    auto and_row = [&](LaneWords<LW> &acc, uint32_t byte_offset) {
        LaneWords<LW> r;
        r.load(col + byte_offset);
#pragma unroll
        for (int u = 0; u < LW; ++u) acc.w[u] &= r.w[u];
    };

    auto evaluate = [&](const Chunk32 &head, const uint32_t *list, const int32_t *weights_of_clause) {
        const int my_weight = pair_lane ? weights_of_clause[my_k] : 0;  // needed only if the clause fires
        const int nb = (int)head.v[0];
        LaneWords<LW> acc;
#pragma unroll
        for (int u = 0; u < LW; ++u) acc.w[u] = active ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int i = 1; i < 8; ++i) and_row(acc, head.v[i]);
        // stop as soon as the clause is false at every node slot of the tile
        if (nb > 1 && __ballot(any_bit(acc)) != 0) {
            // entries past the first chunk, 16 at a time, requested one step before they are needed
            const Chunk16 *tp = reinterpret_cast<const Chunk16 *>(list) + 2;
            Chunk16 tail = *tp;
#pragma unroll
            for (int i = 8; i < 16; ++i) and_row(acc, head.v[i]);
            if (nb > 2 && __ballot(any_bit(acc)) != 0) {
#pragma unroll
                for (int i = 16; i < 24; ++i) and_row(acc, head.v[i]);
                if (nb > 3 && __ballot(any_bit(acc)) != 0) {
#pragma unroll
                    for (int i = 24; i < 32; ++i) and_row(acc, head.v[i]);
                    for (int j = 4; j < nb && __ballot(any_bit(acc)) != 0; j += 2) {
                        const Chunk16 ahead = *++tp;
#pragma unroll
                        for (int i = 0; i < 8; ++i) and_row(acc, tail.v[i]);
                        if (j + 1 < nb && __ballot(any_bit(acc)) != 0) {
#pragma unroll
                            for (int i = 8; i < 16; ++i) and_row(acc, tail.v[i]);
                        }
                        tail = ahead;
                    }
                }
            }
        }
        const unsigned long long nz = __ballot(any_bit(acc));
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

    // Two clauses per trip so that the chunk fetched ahead never has to be
    // copied.  Pointers step by NWAVES clauses; past the end they stay on the
    // wave's last clause (a valid address whose data is not used).
    const int64_t list_step = (int64_t)NWAVES * stride;
    const int wt_step = NWAVES * K;
    const int first = wave < C ? wave : 0;
    const uint32_t *list_a = lists + (int64_t)first * stride;
    const int32_t *wt_a = wt + (int64_t)first * K;
    Chunk32 a = *reinterpret_cast<const Chunk32 *>(list_a);
    for (int c = wave; c < C; c += 2 * NWAVES) {
        const bool has_b = c + NWAVES < C;
        const uint32_t *list_b = has_b ? list_a + list_step : list_a;
        const int32_t *wt_b = has_b ? wt_a + wt_step : wt_a;
        const Chunk32 b = *reinterpret_cast<const Chunk32 *>(list_b);
        evaluate(a, list_a, wt_a);
        const bool has_a = c + 2 * NWAVES < C;
        list_a = has_a ? list_b + list_step : list_b;
        wt_a = has_a ? wt_b + wt_step : wt_b;
        a = *reinterpret_cast<const Chunk32 *>(list_a);
        if (has_b) evaluate(b, list_b, wt_b);
    }
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NWAVES * 64) {
        int64_t g = g0 + i / K;
        if (g >= first_graph && g < (int64_t)first_graph + n_graphs)
            class_sum[(g - first_graph) * K + (i % K)] = sums[i];
    }
}
