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
//   whole number of 32-bit words.
#pragma once

struct TileGeom {
    int slot_bits;   // bits per graph slot
    int slot_words;  // words per graph slot (0 when slot_bits < 32)
    int gpt;         // graphs per tile
    int tw;          // words per tile row (<= 64)
    int rows;        // LITERALS + node types + 1
    int n_tiles;
    int ok;          // geometry supported by the fused kernel
};

constexpr int TILE_MAX_WORDS = 64;
constexpr size_t TILE_LDS_BUDGET = 156 * 1024;  // of the 160 KB per CU

inline TileGeom tile_geometry(int literals, int n_types, int max_nodes, int n_graphs, int classes) {
    TileGeom g{};
    if (max_nodes < 1) max_nodes = 1;
    if (max_nodes <= 16) {
        int s = 1;
        while (s < max_nodes) s <<= 1;
        g.slot_bits = s;
        g.slot_words = 0;
        g.tw = TILE_MAX_WORDS;
        g.gpt = TILE_MAX_WORDS * 32 / s;
    } else {
        g.slot_words = (max_nodes - 1) / 32 + 1;
        g.slot_bits = g.slot_words * 32;
        g.gpt = g.slot_words <= TILE_MAX_WORDS ? TILE_MAX_WORDS / g.slot_words : 0;
        g.tw = g.gpt * g.slot_words;
    }
    g.rows = literals + n_types + 1;
    g.n_tiles = g.gpt > 0 ? (n_graphs + g.gpt - 1) / g.gpt : 0;
    size_t lds = (size_t)g.rows * g.tw * 4 + (size_t)g.gpt * classes * 4;
    g.ok = g.gpt > 0 && lds <= TILE_LDS_BUDGET && literals < 65535 - 8;
    return g;
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
        out = 0xFFFFFFFFu;
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

// Per call, one wave per clause: the clause's included literals as a list of
// 16-bit LDS word offsets (row * tw) in blocks of 8 entries (one 16-byte scalar
// load each).  Entry 0 of the first block is the number of blocks; unused
// entries point at the all-ones row.  The literals are emitted in `order`, so
// the ones that hold least often come first and the running AND dies (and the
// walk stops) as early as it can; the order does not change the result.  Also
// the weights clause-major.
__global__ void k_compile_clauses(const uint32_t *__restrict__ bank, int C, int LA, int B, uint32_t filter, int K,
                                  const int32_t *__restrict__ weights, int literals, int ones_row, int tw,
                                  int stride, const uint32_t *__restrict__ order, uint16_t *__restrict__ lists,
                                  int32_t *__restrict__ wt) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (c >= C) return;
    uint16_t *list = lists + (int64_t)c * stride;
    const uint32_t *inc = bank + (int64_t)c * LA * B + (B - 1);
    int n = 1;  // entry 0 is the header
    for (int r0 = 0; r0 < literals; r0 += 64) {
        int r = r0 + lane;
        uint32_t lit = r < literals ? order[r] : 0u;
        uint32_t w = lit >> 5;
        uint32_t word = inc[(int64_t)w * B];
        if ((int)w == LA - 1) word &= filter;
        bool included = r < literals && ((word >> (lit & 31)) & 1u);
        unsigned long long mask = __ballot(included);
        if (included) list[n + __popcll(mask & ((1ull << lane) - 1ull))] = (uint16_t)(lit * tw);
        n += __popcll(mask);
    }
    const int padded = (n + 7) & ~7;
    for (int i = n + lane; i < padded + 8; i += 64) list[i] = (uint16_t)(ones_row * tw);  // + one block of slack
    if (lane == 0) list[0] = (uint16_t)(padded >> 3);
    for (int k = lane; k < K; k += 64) wt[(int64_t)c * K + k] = weights[(int64_t)k * C + c];
}

__device__ __forceinline__ uint32_t and8(uint32_t acc, const uint32_t *col, uint4 ids, bool skip_first) {
    if (!skip_first) acc &= col[ids.x & 0xFFFFu];
    acc &= col[ids.x >> 16];
    acc &= col[ids.y & 0xFFFFu];
    acc &= col[ids.y >> 16];
    acc &= col[ids.z & 0xFFFFu];
    acc &= col[ids.z >> 16];
    acc &= col[ids.w & 0xFFFFu];
    acc &= col[ids.w >> 16];
    return acc;
}

// One workgroup per tile.  The tile's bit-rows are copied to LDS once; each
// wave then walks its share of the clauses.  The clause id and its literal
// list are wave-uniform (scalar loads, issued one block ahead); lane L holds
// word L of the running AND.
template <int NWAVES>
__global__ __launch_bounds__(NWAVES * 64) void k_score_tiles(
    const uint32_t *__restrict__ tiles, TileGeom tg, int literals, int n_types, int C, int K,
    const uint16_t *__restrict__ lists, int stride, const int32_t *__restrict__ wt, int tile0, int first_graph,
    int n_graphs, int32_t *__restrict__ class_sum) {
    extern __shared__ uint32_t lds[];
    const int tw = tg.tw;
    uint32_t *bt = lds;
    int32_t *sums = (int32_t *)(lds + (size_t)tg.rows * tw);
    const int tile = tile0 + blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    const uint32_t *src = tiles + (int64_t)tile * tg.rows * tw;
    for (int i = tid; i < tg.rows * tw; i += NWAVES * 64) bt[i] = src[i];
    for (int i = tid; i < tg.gpt * K; i += NWAVES * 64) sums[i] = 0;
    __syncthreads();

    const bool active = lane < tw;
    const uint32_t *col = bt + (active ? lane : 0);
    const int stride4 = stride >> 3;  // list stride in 16-byte blocks
    const uint4 *all = reinterpret_cast<const uint4 *>(lists);

    // lane p < gpt*K adds weight k = p % K to graph j = p / K of the tile
    const int pairs = tg.gpt * K;
    const int my_j = lane / K, my_k = lane - my_j * K;
    const bool pair_lane = tg.slot_words > 0 && lane < pairs;
    const int my_shift = (lane < tg.gpt ? lane : 0) * tg.slot_words;
    const unsigned long long slot_lanes = tg.slot_words >= 64 ? ~0ull : (1ull << tg.slot_words) - 1ull;

    int c = wave;
    int type_row = literals + c % n_types;
    const int type_step = NWAVES % n_types;
    uint4 head = all[(int64_t)(c < C ? c : 0) * stride4];
    while (c < C) {
        const int cn = c + NWAVES;
        const uint4 *lp = all + (int64_t)c * stride4;
        const uint4 head_next = all[(int64_t)(cn < C ? cn : c) * stride4];  // next clause, fetched early
        uint4 block = lp[1];
        const int my_weight = pair_lane ? wt[(int64_t)c * K + my_k] : 0;  // needed only if the clause fires
        const int nb = head.x & 0xFFFFu;
        uint32_t acc = active ? col[type_row * tw] : 0u;
        type_row += type_step;
        if (type_row >= literals + n_types) type_row -= n_types;
        acc = and8(acc, col, head, true);
        for (int j = 1; j < nb; ++j) {
            const uint4 ahead = lp[j + 1];
            if (__ballot(acc != 0) == 0) break;  // false at every node slot of the tile
            acc = and8(acc, col, block, false);
            block = ahead;
        }
        const unsigned long long nz = __ballot(acc != 0);
        if (nz != 0) {
            if (tg.slot_words > 0) {
                // graph j owns lanes [j*slot_words, (j+1)*slot_words)
                const unsigned long long gm = __ballot(lane < tg.gpt && ((nz >> my_shift) & slot_lanes) != 0);
                if (pair_lane && ((gm >> my_j) & 1ull)) atomicAdd(&sums[lane], my_weight);
                for (int p = lane + 64; p < pairs; p += 64) {
                    int j = p / K, k = p - j * K;
                    if ((gm >> j) & 1ull) atomicAdd(&sums[p], wt[(int64_t)c * K + k]);
                }
            } else {
                // several graphs per word: walk the non-empty slots of this lane's word
                const int per_word = 32 / tg.slot_bits;
                const uint32_t slot_mask = (1u << tg.slot_bits) - 1u;  // slot_bits <= 16
                while (acc) {
                    int sub = (__ffs(acc) - 1) / tg.slot_bits;
                    acc &= ~(slot_mask << (sub * tg.slot_bits));
                    int j = lane * per_word + sub;
                    for (int k = 0; k < K; ++k) atomicAdd(&sums[j * K + k], wt[(int64_t)c * K + k]);
                }
            }
        }
        head = head_next;
        c = cn;
    }
    __syncthreads();
    const int64_t g0 = (int64_t)tile * tg.gpt;
    for (int i = tid; i < tg.gpt * K; i += NWAVES * 64) {
        int64_t g = g0 + i / K;
        if (g >= first_graph && g < (int64_t)first_graph + n_graphs)
            class_sum[(g - first_graph) * K + (i % K)] = sums[i];
    }
}
