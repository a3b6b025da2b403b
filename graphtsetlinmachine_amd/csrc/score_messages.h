// The message rows of a layer, one TILE per workgroup, with everything between the truth rows
// and the literal-major rows kept in LDS (graphs too big for k_tile_messages_fused, whose two sets
// of vectors per graph must both fit: a graph of 841 nodes with messages of 1,024 bits).
//
// A message factors (kernels.py:565-588): what a node sends is the OR of the hypervector bits of
// the clauses true at it, and what a neighbour receives along an edge of type t is that vector
// rotated by t.  Four steps on one region of LDS:
//   1. rows[p] |= truth row of every clause whose hypervector holds bit p: M rows of tw words,
//      LDS atomics.  Each truth row is read ONCE (a quarter-wave per clause, 8 bytes per lane), and only the rows of the clauses that the
//      evaluation listed as true somewhere in the tile when such lists are handed in;
//   2. the M x (32 tw) bit matrix is turned node-major in place - every half-wave takes 32 x 32
//      bit blocks through registers (a transposition across its lanes), all blocks are read
//      before any is written back: slot n's vector of MW words now starts at n (MW + 1);
//   3. along the edges, a range of destination slots at a time (as many as the LDS left over
//      holds): every thread owns a source slot and ORs its vector, rotated by the edge's type,
//      into the vectors of its destinations inside the range (LDS atomics; the edges of a node
//      come from global memory once, the first four stay in registers);
//   4. the range's received vectors are turned literal-major, 32 x 32 bits per half-wave again,
//      and stored, 16 bytes per lane, as words of the rows [M + 2][tw] that the next layer's
//      evaluation stages.
// No vector ever goes to global memory and nothing is cleared there.
#pragma once

#include <type_traits>

constexpr int TILE_MESSAGES_LDS_BLOCK = 1024;

// The word of lane `from` (0 .. 15) of this lane's row of 16 lanes: a lane move on the vector unit.  (`from` is
// a constant wherever this is called - an unrolled loop's counter - and the switch folds away.)
__device__ __forceinline__ uint32_t tile_row_share(uint32_t v, int from) {
    switch (from & 15) {
#define GTM_ROW_SHARE(n) \
    case n: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x150 + n, 0xF, 0xF, true);
        GTM_ROW_SHARE(0) GTM_ROW_SHARE(1) GTM_ROW_SHARE(2) GTM_ROW_SHARE(3) GTM_ROW_SHARE(4) GTM_ROW_SHARE(5)
        GTM_ROW_SHARE(6) GTM_ROW_SHARE(7) GTM_ROW_SHARE(8) GTM_ROW_SHARE(9) GTM_ROW_SHARE(10) GTM_ROW_SHARE(11)
        GTM_ROW_SHARE(12) GTM_ROW_SHARE(13) GTM_ROW_SHARE(14)
#undef GTM_ROW_SHARE
    default: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x15F, 0xF, 0xF, true);
    }
}

struct TileMessagesPlan {
    int ok;
    int main_words;   // LDS words of the region that holds the rows, then the vectors
    int range_words;  // words of destination slots (32 each) whose received vectors fit beside it
    size_t lds_bytes;
};

// Shapes the kernel takes: M a multiple of 32 and at most 1,024, tiles of at most 64 words (one or two node slots
// per thread), at most 1,024 blocks of 32 x 32 bits in the rows, and room in LDS for the vectors plus at least
// 128 received ones.
inline TileMessagesPlan tile_messages_lds_plan(const TileGeom &g, int M, size_t lds_limit) {
    TileMessagesPlan p{};
    if (!g.ok || M < 32 || M % 32 != 0 || M > 1024 || g.tw > 64 || g.tw % 4 != 0) return p;
    const int MW = M / 32;
    if (MW * g.tw > 1024) return p;
    const size_t rows = (size_t)M * g.tw, vectors = (size_t)g.tw * 32 * (MW + 1);
    const size_t main_words = rows > vectors ? rows : vectors;
    const size_t per_word = (size_t)32 * (MW + 1);
    if ((main_words + 4 * per_word) * 4 > lds_limit) return p;
    size_t range = (lds_limit / 4 - main_words) / per_word & ~(size_t)3;  // (rows are stored four words at a time)
    if (range > (size_t)g.tw) range = (size_t)g.tw;
    p.ok = 1;
    p.main_words = (int)main_words;
    p.range_words = (int)range;
    p.lds_bytes = (main_words + range * per_word) * 4;
    return p;
}

// WIDE: rows of 33 to 64 words - a quarter-wave reads a truth row at four words per lane, and a thread owns two
// node slots.
template <bool WIDE>
__global__ __launch_bounds__(TILE_MESSAGES_LDS_BLOCK) void k_tile_messages_in_lds(
    const uint32_t *__restrict__ bitmap, int C, TileGeom tg, int tile0, int G, int M, const uint32_t *__restrict__ hv, int MB,
    const uint32_t *__restrict__ alive, int streams, int alive_stride, const uint32_t *__restrict__ node_index,
    const uint32_t *__restrict__ n_nodes, const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
    const uint32_t *__restrict__ edge, int has_edges, int main_words, int range_words, uint32_t *__restrict__ rows) {
    extern __shared__ uint32_t lds[];
    constexpr int NT = TILE_MESSAGES_LDS_BLOCK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile_local = blockIdx.x;
    const int tw = tg.tw, MW = M >> 5, VS = MW + 1, S = tw * 32;
    uint32_t *main_region = lds;
    uint32_t *got = lds + main_words;
    uint32_t *out = rows + (int64_t)tile_local * (M + 2) * tw;

    for (int i = tid; i < M * tw; i += NT) main_region[i] = 0u;
    __syncthreads();

    // 1. the rows of what is sent, literal-major.  Lane l of a quarter-wave fetches the number and the first two
    // hypervector bits of the stream's clause 16 k + l, a group of 16 clauses ahead of the truth rows; a clause's
    // number and bits then reach the 16 lanes by a lane move (row_share), and eight truth rows are on their way
    // per quarter-wave.
    {
        constexpr int WPL = WIDE ? 4 : 2;  // words of a truth row per lane
        typedef uint32_t Words __attribute__((ext_vector_type(WPL)));
        const int group = lane >> 4, gl = lane & 15;
        // the tile's truth rows through a buffer descriptor: a row is reached by a multiply-add of 24-bit factors per
        // lane (clause x bytes per row + the lane's place), not by a 64-bit multiply and add
        const __amdgpu_buffer_rsrc_t truth = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint32_t *>(bitmap + (int64_t)tile_local * C * tw), 0, C * tw * 4, 0x00020000);
        const bool has_words = WPL * gl < tw;
        const uint32_t place = has_words ? 4u * WPL * gl : 0u;
        // a quarter-wave takes the streams q, q + 64, ... of the evaluation that wrote the truth rows
        for (int q = wave * 4 + group; q < streams; q += TILE_MESSAGES_LDS_BLOCK / 16) {
        const uint32_t *list = alive ? alive + ((int64_t)tile_local * streams + q) * alive_stride : nullptr;
        const int n_mine = list ? (int)list[0] : (q < C ? (C - q + streams - 1) / streams : 0);
        uint32_t id_next = 0u, bit0_next = 0u, bit1_next = 0u;
        // (every load below is unconditional, from an address that exists, and what it brought is dropped
        // afterwards where it was not wanted: loads under a condition would wait for one another)
        auto fetch = [&](int i) {
            const int at = i < n_mine ? i : n_mine - 1;
            id_next = list ? list[1 + at] : (uint32_t)(q + streams * at);
            bit0_next = hv[(int64_t)id_next * MB];
            bit1_next = hv[(int64_t)id_next * MB + (MB > 1 ? 1 : 0)];
        };
        if (n_mine > 0) fetch(gl);
        for (int i0 = 0; i0 < n_mine; i0 += 16) {  // (the lanes of a quarter-wave leave the loop together)
            const uint32_t id = id_next, bit0 = bit0_next, bit1 = bit1_next;
            fetch(i0 + 16 + gl);
            const int n_here = n_mine - i0 < 16 ? n_mine - i0 : 16;
            auto eight = [&](auto first_of_eight) {  // clauses u0 .. u0 + 7 of the 16
                constexpr int u0 = decltype(first_of_eight)::value;
                uint32_t c[8];
                Words t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    c[u] = tile_row_share(id, u0 + u);  // (past the stream's end: its last clause once more)
                    const int at = (int)(__umul24(c[u], (uint32_t)tw * 4u) + place);
                    if constexpr (WIDE) {
                        t[u] = __builtin_amdgcn_raw_buffer_load_b128(truth, at, 0, 0);
                    } else {
                        t[u] = __builtin_amdgcn_raw_buffer_load_b64(truth, at, 0, 0);
                    }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const uint32_t h0 = tile_row_share(bit0, u0 + u), h1 = tile_row_share(bit1, u0 + u);
                    uint32_t any = t[u][0] | t[u][1];
                    if (WIDE) any |= t[u][2] | t[u][3];
                    if (u0 + u >= n_here || !has_words || any == 0u) continue;
                    for (int j = 0; j < MB; ++j) {
                        const uint32_t h = j == 0 ? h0 : j == 1 ? h1 : hv[(int64_t)c[u] * MB + j];
                        if (h >= (uint32_t)M) continue;
                        // (tw is a multiple of 4: each pair of words is one aligned 64-bit word of LDS)
                        unsigned long long *row = reinterpret_cast<unsigned long long *>(main_region + __umul24(h, (uint32_t)tw) + WPL * gl);
#pragma unroll
                        for (int v = 0; v < WPL / 2; ++v) {
                            const unsigned long long both =
                                (unsigned long long)t[u][2 * v] | ((unsigned long long)t[u][2 * v + 1] << 32);
                            if (both) atomicOr(&row[v], both);
                        }
                    }
                }
            };
            eight(std::integral_constant<int, 0>{});
            if (n_here > 8) eight(std::integral_constant<int, 8>{});
        }
        }
    }
    __syncthreads();

    // 2. node-major in place: block (j, w) - rows 32 j .. 32 j + 31, word w - becomes word j of slots 32 w .. 32 w + 31
    const int hw = tid >> 5, hl = lane & 31;
    {
        const int n_blocks = MW * tw;
        // block k * 32 + hw is (j, w) = (id / tw, id % tw): one division, then steps of 32 blocks
        const int step_j = 32 / tw, step_w = 32 - step_j * tw;
        const int j_first = hw / tw, w_first = hw - j_first * tw;
        uint32_t held[32];
        int j = j_first, w = w_first;
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            held[k] = 0u;
            if (k * 32 >= n_blocks) continue;  // (the same for every thread)
            const int id = k * 32 + hw;
            uint32_t v = 0u;
            if (id < n_blocks) v = main_region[(32 * j + hl) * tw + w];
            held[k] = tile_transpose32(v, lane);
            j += step_j, w += step_w;
            if (w >= tw) w -= tw, ++j;
        }
        __syncthreads();
        j = j_first, w = w_first;
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int id = k * 32 + hw;
            if (id < n_blocks) main_region[(32 * w + hl) * VS + j] = held[k];
            j += step_j, w += step_w;
            if (w >= tw) w -= tw, ++j;
        }
    }

    // the all-ones row and the row of graphs without nodes (slot bit 0 of each: kernels.py:443-466,505-527 leave every
    // clause true for such a graph at every layer, which the message literals must not undo)
    for (int w = tid; w < tw; w += NT) {
        const int used = tg.slot_words == 0 ? tw : tg.gpt * tg.slot_words;
        uint32_t empties = 0u;
        for (int b = 0; b < 32; ++b) {
            const int pos = w * 32 + b, gj = pos / tg.slot_bits;
            const int64_t g = (int64_t)(tile0 + tile_local) * tg.gpt + gj;
            if (pos == gj * tg.slot_bits && gj < tg.gpt && g < G && n_nodes[g] == 0u) empties |= 1u << b;
        }
        out[(int64_t)M * tw + w] = w < used ? 0xFFFFFFFFu : 0u;
        out[(int64_t)(M + 1) * tw + w] = empties;
    }

    // this thread's source slots (tid, and tid + 1,024 on rows of more than 32 words) and their edges
    constexpr int SPT = WIDE ? 2 : 1;
    uint32_t ne[SPT], nodes_of_graph[SPT];
    int slot0[SPT];
    const uint2 *out_edges[SPT];
    uint2 first[SPT][4];
    const uint32_t *mine[SPT];
#pragma unroll
    for (int h = 0; h < SPT; ++h) {
        const int slot = tid + h * NT;
        ne[h] = 0u, nodes_of_graph[h] = 0u, slot0[h] = 0, out_edges[h] = nullptr;
        if (slot < S && has_edges) {
            const int gj = slot / tg.slot_bits, n = slot - gj * tg.slot_bits;
            const int64_t g = (int64_t)(tile0 + tile_local) * tg.gpt + gj;
            if (gj < tg.gpt && g < G && (uint32_t)n < n_nodes[g]) {
                const int64_t row = (int64_t)node_index[g] + n;
                ne[h] = n_edges[row];
                out_edges[h] = reinterpret_cast<const uint2 *>(edge) + edge_index[row];
                nodes_of_graph[h] = n_nodes[g];
                slot0[h] = gj * tg.slot_bits;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            first[h][u] = (uint32_t)u < ne[h] ? out_edges[h][u] : make_uint2(0u, 0u);
            first[h][u].y %= (uint32_t)M;  // (the edge's rotation, reduced once for all the passes)
        }
        mine[h] = main_region + (slot < S ? slot : 0) * VS;
    }

    for (int w_lo = 0; w_lo < tw; w_lo += range_words) {
        const int w_hi = w_lo + range_words < tw ? w_lo + range_words : tw, nw = w_hi - w_lo;
        for (int i = tid; i < nw * 32 * VS; i += NT) got[i] = 0u;
        __syncthreads();  // (also: every vector of step 2 is in place)

        // 3. along the edges into the range: bit p of what arrives is bit (p - shift) mod M of what was sent, so word
        // j of the node's vector, moved up by r = shift % 32 bits with the top of word j - 1 below it, lands in word
        // (j + shift / 32) mod MW.  A word of the vector is read once for the (up to four) edges at hand, and the
        // move is one 64-bit shift of (word j, word j - 1) by 32 - r.
#pragma unroll
        for (int h = 0; h < SPT; ++h)
            for (uint32_t e0 = 0; e0 < ne[h]; e0 += 4) {
                uint32_t *to[4];
                uint32_t down[4];
                int at[4];
                bool on[4], any = false;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    uint2 pair = first[h][u];
                    if (e0 != 0) {
                        pair = e0 + u < ne[h] ? out_edges[h][e0 + u] : make_uint2(0u, 0u);
                        pair.y %= (uint32_t)M;
                    }
                    const uint32_t dst = pair.x;
                    const int to_slot = slot0[h] + (int)dst, to_word = to_slot >> 5;
                    on[u] = e0 + u < ne[h] && dst < nodes_of_graph[h] && to_word >= w_lo && to_word < w_hi;
                    to[u] = got + (on[u] ? to_slot - 32 * w_lo : 0) * VS;
                    down[u] = 32u - (pair.y & 31u);
                    at[u] = (int)(pair.y >> 5);
                    any = any || on[u];
                }
                if (!any) continue;
                uint32_t below = mine[h][MW - 1];
                for (int j = 0; j < MW; ++j) {
                    const uint32_t cur = mine[h][j];
                    const unsigned long long both = ((unsigned long long)cur << 32) | below;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint32_t word = (uint32_t)(both >> down[u]);
                        if (on[u] && word) atomicOr(&to[u][at[u]], word);
                        at[u] = at[u] + 1 == MW ? 0 : at[u] + 1;
                    }
                    below = cur;
                }
            }
        __syncthreads();

        // 4. literal-major: block (j, w) of the range - word j of slots 32 w .. 32 w + 31 - becomes word w of rows
        // 32 j .. 32 j + 31; a half-wave turns four neighbouring blocks and each lane stores its row's four words at once
        const int nq = nw >> 2, n_units = MW * nq;
        const int unit_step_j = 32 / nq, unit_step_w = 32 - unit_step_j * nq;  // (unit k * 32 + hw is (id / nq, id % nq))
        int j = hw / nq, wq = hw - j * nq;
        for (int k = 0; k * 32 < n_units; ++k, j += unit_step_j, wq += unit_step_w) {
            if (wq >= nq) wq -= nq, ++j;
            const int id = k * 32 + hw;
            uint32_t column[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t v = id < n_units ? got[(32 * (4 * wq + u) + hl) * VS + j] : 0u;
                column[u] = tile_transpose32(v, lane);
            }
            if (id < n_units)
                *reinterpret_cast<uint4 *>(out + (int64_t)(32 * j + hl) * tw + w_lo + 4 * wq) =
                    make_uint4(column[0], column[1], column[2], column[3]);
        }
        __syncthreads();
    }
}
