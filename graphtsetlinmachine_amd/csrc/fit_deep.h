// The message layers of one training step (tm.py:595-650) for one graph.
//
//   k_fit_scatter_messages  K4 (+K5): one thread per (clause, node); a clause
//                           that is true at the node sets, at every
//                           out-neighbour, its hypervector bits rotated by the
//                           edge type and clears their negations, straight into
//                           the packed node-major message words (blanked first
//                           by k_messages_blank, K3).
//   k_fit_message_rows      the positive half of those words turned literal-
//                           major: row p holds bit p of every node.
//   k_fit_message_eval      K2: as k_fit_eval, but a clause starts from its
//                           truth in the layer before and ANDs the message rows
//                           (or their complements, for negated message
//                           literals) that its message automata include.
#pragma once

constexpr int FIT_SCATTER_BLOCK = 256;

__global__ __launch_bounds__(FIT_SCATTER_BLOCK) void k_fit_scatter_messages(
    const uint32_t *__restrict__ bitmap, int C, int NC, int n_nodes, const uint32_t *__restrict__ hv, int MB, int M,
    int MC, const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
    const uint32_t *__restrict__ edge, uint32_t *clause_X) {
    // n_edges / edge_index point at the graph's first node
    const int64_t i = (int64_t)blockIdx.x * FIT_SCATTER_BLOCK + threadIdx.x;
    const int c = (int)(i / n_nodes), n = (int)(i - (int64_t)c * n_nodes);
    if (c >= C) return;
    if (!((bitmap[(int64_t)c * NC + (n >> 5)] >> (n & 31)) & 1u)) return;
    const uint32_t ne = n_edges[n];
    const int64_t e0 = edge_index[n];
    for (uint32_t e = 0; e < ne; ++e) {
        const uint32_t dst = edge[(e0 + e) * 2], type = edge[(e0 + e) * 2 + 1];
        for (int j = 0; j < MB; ++j) {
            const uint32_t pos = (hv[(int64_t)c * MB + j] + type) % (uint32_t)M;
            const uint32_t neg = pos + (uint32_t)M;
            atomicOr(&clause_X[(int64_t)dst * MC + (pos >> 5)], 1u << (pos & 31));
            atomicAnd(&clause_X[(int64_t)dst * MC + (neg >> 5)], ~(1u << (neg & 31)));
        }
    }
}

// One wave per (32 message literals, 64 nodes): lane n holds the node's word of
// those literals; the ballot of bit b over the wave is row 32w + b for these 64
// nodes.  rows[M][row_words], row_words even.
__global__ __launch_bounds__(64) void k_fit_message_rows(const uint32_t *__restrict__ clause_X, int n_nodes, int M,
                                                          int MC, int row_words, uint32_t *__restrict__ rows) {
    const int lane = threadIdx.x;
    const int w = blockIdx.x, nb = blockIdx.y;
    const int n = nb * 64 + lane;
    const uint32_t word = n < n_nodes ? clause_X[(int64_t)n * MC + w] : 0u;
    unsigned long long mine = 0;
#pragma unroll
    for (int b = 0; b < 32; ++b) {
        const unsigned long long column = __ballot((word >> b) & 1u);
        if (lane == b) mine = column;
    }
    const int p = w * 32 + lane;
    if (lane < 32 && p < M) {
        rows[(int64_t)p * row_words + nb * 2] = (uint32_t)mine;
        rows[(int64_t)p * row_words + nb * 2 + 1] = (uint32_t)(mine >> 32);
    }
}

// ---- messages in three steps, for MESSAGE_SIZE a multiple of 32 -------------
//
// A message (kernels.py:565-588) factors: the bits a node sends are the OR of
// the hypervector bits of the clauses true at it, and what a neighbour receives
// along an edge of type t is that bit vector rotated by t.  So:
//   k_fit_node_messages  sent[n] = OR over clauses true at n of their bits
//   k_fit_edge_messages  got[dst] |= rotate(sent[src], type) for every edge
//   k_fit_pack_messages  node-major packed literals (got | ~got) and the
//                        literal-major rows of got; clears sent and got
// which needs (true pairs x MESSAGE_BITS) LDS atomics and (edges x words)
// global ones instead of (true pairs x edges x MESSAGE_BITS x 2) global ones.

constexpr int FIT_NODE_MESSAGES_BLOCK = 1024;
constexpr int FIT_NODE_MESSAGES_CLAUSES = 1024;  // clauses per block
constexpr int FIT_NODE_MESSAGES_PARTS = 4;       // threads that share a clause's word of 32 nodes

// grid (node words in use, ceil(C / FIT_NODE_MESSAGES_CLAUSES)); dynamic LDS 32 * (MW | 1) words.
// What a thread does is a chain of dependent LDS atomics, so a clause's 32 nodes are split over
// FIT_NODE_MESSAGES_PARTS threads, and a hypervector bit is fetched once for all of a thread's nodes.
__global__ __launch_bounds__(FIT_NODE_MESSAGES_BLOCK) void k_fit_node_messages(
    const uint32_t *__restrict__ bitmap, int C, int NC, int n_nodes, const uint32_t *__restrict__ hv, int MB, int MW,
    uint32_t *sent, const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
    const uint32_t *__restrict__ edge, uint32_t *got) {
    extern __shared__ uint32_t vec[];  // [32 nodes][MW | 1]: lanes on different nodes hit different banks
    const int tid = threadIdx.x;
    const int nw = blockIdx.x;
    const int MWP = MW | 1;
    constexpr int PARTS = FIT_NODE_MESSAGES_PARTS, BITS = 32 / PARTS;
    for (int i = tid; i < 32 * MWP; i += FIT_NODE_MESSAGES_BLOCK) vec[i] = 0u;
    __syncthreads();
    const int c_end = min(C, (int)(blockIdx.y + 1) * FIT_NODE_MESSAGES_CLAUSES);
    const uint32_t valid = n_nodes - nw * 32 >= 32 ? 0xFFFFFFFFu : (1u << (n_nodes - nw * 32)) - 1u;
    const uint32_t mine = valid & (((1u << BITS) - 1u) << ((tid % PARTS) * BITS));
    for (int c = blockIdx.y * FIT_NODE_MESSAGES_CLAUSES + tid / PARTS; c < c_end; c += FIT_NODE_MESSAGES_BLOCK / PARTS) {
        const uint32_t word = bitmap[(int64_t)c * NC + nw] & mine;
        if (!word) continue;
        for (int j = 0; j < MB; ++j) {
            const uint32_t h = hv[(int64_t)c * MB + j];
            uint32_t *column = vec + (h >> 5);
            const uint32_t bit = 1u << (h & 31);
            for (uint32_t m = word; m; m &= m - 1) atomicOr(&column[(__ffs(m) - 1) * MWP], bit);
        }
    }
    __syncthreads();
    if (n_edges != nullptr) {
        // One block holds every clause (the host passes the edges only then): its 32 vectors are
        // complete and go along the edges from here, as k_fit_edge_messages would send them.
        const uint32_t M = (uint32_t)MW * 32u;
        for (int i = tid; i < 32 * MW; i += FIT_NODE_MESSAGES_BLOCK) {
            const int nl = i / MW, j = i - nl * MW, n = nw * 32 + nl;
            if (n >= n_nodes) continue;
            const uint32_t *v = vec + nl * MWP;
            const uint32_t ne = n_edges[n];
            const int64_t e0 = edge_index[n];
            for (uint32_t e = 0; e < ne; ++e) {
                const uint32_t dst = edge[(e0 + e) * 2], shift = edge[(e0 + e) * 2 + 1] % M;
                const int q = (int)(shift >> 5), r = (int)(shift & 31u);
                const int a = (j - q + MW) % MW, below = (a - 1 + MW) % MW;
                const uint32_t word = r ? (v[a] << r) | (v[below] >> (32 - r)) : v[a];
                if (word) atomicOr(&got[(int64_t)dst * MW + j], word);
            }
        }
        return;
    }
    for (int i = tid; i < 32 * MW; i += FIT_NODE_MESSAGES_BLOCK) {
        const int n = nw * 32 + i / MW;
        const uint32_t word = vec[(i / MW) * MWP + i % MW];
        if (word != 0u && n < n_nodes) atomicOr(&sent[(int64_t)n * MW + (i % MW)], word);
    }
}

// One thread per (node, word of the rotated vector): for each of the node's
// out-edges, word j of rotate(sent[node], type) ORed into got[destination].
__global__ void k_fit_edge_messages(const uint32_t *__restrict__ sent, int n_nodes, int MW,
                                    const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
                                    const uint32_t *__restrict__ edge, uint32_t *got) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)n_nodes * MW) return;
    const int n = (int)(i / MW), j = (int)(i % MW);
    const uint32_t *v = sent + (int64_t)n * MW;
    const uint32_t ne = n_edges[n];
    const int64_t e0 = edge_index[n];
    const uint32_t M = (uint32_t)MW * 32u;
    for (uint32_t e = 0; e < ne; ++e) {
        const uint32_t dst = edge[(e0 + e) * 2], shift = edge[(e0 + e) * 2 + 1] % M;
        // bit p of the result is bit (p - shift) mod M of v
        const int q = (int)(shift >> 5), r = (int)(shift & 31u);
        const int a = (j - q + MW) % MW, below = (a - 1 + MW) % MW;
        const uint32_t word = r ? (v[a] << r) | (v[below] >> (32 - r)) : v[a];
        if (word) atomicOr(&got[(int64_t)dst * MW + j], word);
    }
}

// One wave per (word j of the message vectors, 64 nodes), lane = node: writes
// the node's packed literal words j (messages) and MW + j (their negations),
// the literal-major rows 32 j .. 32 j + 31 for these 64 nodes, and clears the
// node's words of sent and got for the next use.  clause_X is [node][2 * MW].
__global__ __launch_bounds__(64) void k_fit_pack_messages(uint32_t *sent, uint32_t *got, int n_nodes, int MW,
                                                           int row_words, uint32_t *__restrict__ clause_X,
                                                           uint32_t *__restrict__ rows) {
    const int lane = threadIdx.x;
    const int j = blockIdx.x, nb = blockIdx.y;
    const int n = nb * 64 + lane;
    uint32_t word = 0u;
    if (n < n_nodes) {
        word = got[(int64_t)n * MW + j];
        got[(int64_t)n * MW + j] = 0u;
        sent[(int64_t)n * MW + j] = 0u;
        clause_X[(int64_t)n * 2 * MW + j] = word;
        clause_X[(int64_t)n * 2 * MW + MW + j] = ~word;
    }
    // each half of the wave transposes its 32 nodes x 32 bits: lane b of a half holds one word of row 32 j + b
    rows[(int64_t)(j * 32 + (lane & 31)) * row_words + nb * 2 + (lane >> 5)] = tile_transpose32(word, lane);
}

// K2 (+ K6 + K7 when `finish`) for one graph and one message layer.  Each block
// takes clauses in turn; lane L ends up with word L of the clause's truth over
// the graph's nodes, starting from the layer before.  The clause's include words
// come from the top bit plane of the layer's automaton bank.  Two ways to apply
// them, chosen per clause by the number of memory round trips each needs:
//   by literal  every included message literal l < M ANDs row l, every l >= M the
//               complement of row l - M (kernels.py:505-527; positions past the
//               graph's nodes are already 0 in the incoming truth);
//   by node     64 nodes at a time, lane = node: the node's packed message words
//               against the clause's include words, (include & ~words) == 0, for
//               the blocks of nodes where the clause is still true.
constexpr int FIT_MESSAGE_EVAL_BLOCK = 1024;  // at most 16 waves: a graph of up to 1,024 nodes has a wave per block of 64 nodes

__global__ __launch_bounds__(FIT_MESSAGE_EVAL_BLOCK) void k_fit_message_eval(
    const uint32_t *__restrict__ rows, int row_words, const uint32_t *__restrict__ clause_X, int words, int n_nodes,
    int M, int C, int MC, int B, int K, int NC, uint32_t filter, const uint32_t *__restrict__ bank,
    const int32_t *__restrict__ weights, uint32_t k0, uint32_t k1, uint32_t step, int finish,
    const uint32_t *__restrict__ bitmap_in, uint32_t *__restrict__ bitmap_out, int32_t *__restrict__ n_incl,
    int32_t *__restrict__ clause_node, int32_t *class_sum) {
    // The waves of a block share a clause: by node they split its blocks of 64 nodes and hand
    // their words to wave 0 through LDS; by literal wave 0 works alone.  Wave 0 ends the clause.
    __shared__ uint32_t handed[64];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int WAVES = (int)(blockDim.x >> 6);  // chosen by the host: few clauses -> many waves per clause
    const bool active = lane < words;
    const uint32_t *col = rows + (active ? lane : 0);
    const bool rows_of_16_bytes = (MC & 3) == 0;  // a node's packed words can be read four at a time
    int partial = 0;
    for (int c = blockIdx.x; c < C; c += gridDim.x) {
        const uint32_t *inc = bank + (int64_t)c * MC * B + (B - 1);
        uint32_t acc = active ? bitmap_in[(int64_t)c * NC + lane] : 0u;
        int included = 0;
        for (int w0 = 0; w0 < MC; w0 += 64) {
            uint32_t mine = w0 + lane < MC ? inc[(int64_t)(w0 + lane) * B] : 0u;
            if (w0 + lane == MC - 1) mine &= filter;
            unsigned long long nonzero = __ballot(mine != 0);
            int here = __popc(mine);
            included += here;
            // words of the truth row that are not zero, and the blocks of 64 nodes they cover
            const unsigned long long live_words = __ballot(acc != 0);
            // a clause that is false everywhere stays false: only its include count is needed
            if (live_words == 0 || nonzero == 0) continue;
            const int live_blocks = __popcll((live_words | (live_words >> 1)) & 0x5555555555555555ull);
            for (int off = 32; off > 0; off >>= 1) here += __shfl_xor(here, off);
            const int trips_by_literal = (here + 7) >> 3;
            const int chunk_words = MC - w0 < 64 ? MC - w0 : 64;
            const int trips_by_node = ((live_blocks + WAVES - 1) / WAVES) *
                                      (rows_of_16_bytes ? (chunk_words + 31) >> 5 : (__popcll(nonzero) + 7) >> 3);
            if (trips_by_node < trips_by_literal) {
                if (tid < 64) handed[tid] = 0u;
                __syncthreads();
                for (int nb = wave; nb * 2 < words; nb += WAVES) {
                    if (((live_words >> (nb * 2)) & 3ull) == 0) continue;
                    const int node = nb * 64 + lane;
                    // this node's bit of the running truth (lane = node)
                    const uint32_t lo = __builtin_amdgcn_readlane(acc, nb * 2);
                    const uint32_t hi = __builtin_amdgcn_readlane(acc, (nb * 2 + 1) & 63);
                    bool ok = ((lane < 32 ? lo >> lane : hi >> (lane - 32)) & 1u) != 0;
                    const uint32_t *x = clause_X + (int64_t)(node < n_nodes ? node : 0) * MC + w0;
                    unsigned long long todo = nonzero;
                    uint32_t violated = 0;
                    if (rows_of_16_bytes) {
                        // the node's words of this chunk, 32 per round trip, against the include words
                        // (zero past the bank's last word, so words read for nothing change nothing)
                        todo = 0ull;
                        const uint4 *x4 = reinterpret_cast<const uint4 *>(x);
                        for (int q0 = 0; q0 * 4 < chunk_words; q0 += 8) {
                            uint4 xs[8];
#pragma unroll
                            for (int u = 0; u < 8; ++u)
                                xs[u] = (q0 + u) * 4 < chunk_words ? x4[q0 + u] : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
                            for (int u = 0; u < 8; ++u) {
                                const int wl = ((q0 + u) * 4) & 63;
                                violated |= (__builtin_amdgcn_readlane(mine, wl) & ~xs[u].x) |
                                            (__builtin_amdgcn_readlane(mine, (wl + 1) & 63) & ~xs[u].y) |
                                            (__builtin_amdgcn_readlane(mine, (wl + 2) & 63) & ~xs[u].z) |
                                            (__builtin_amdgcn_readlane(mine, (wl + 3) & 63) & ~xs[u].w);
                            }
                        }
                    }
                    while (todo) {
                        uint32_t xs[8], is[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const int wl = todo ? __ffsll((long long)todo) - 1 : 0;
                            is[u] = todo ? __builtin_amdgcn_readlane(mine, wl) : 0u;
                            todo &= todo - 1;
                            xs[u] = x[wl];
                        }
#pragma unroll
                        for (int u = 0; u < 8; ++u) violated |= is[u] & ~xs[u];
                    }
                    ok = ok && violated == 0;
                    const unsigned long long truth = __ballot(ok);
                    if (lane == 0) {
                        handed[nb * 2] = (uint32_t)truth;
                        if (nb * 2 + 1 < 64) handed[nb * 2 + 1] = (uint32_t)(truth >> 32);
                    }
                }
                __syncthreads();
                acc = active ? handed[lane] : 0u;  // every wave goes on with the whole row
                __syncthreads();
            } else if (wave == 0) {
                while (nonzero) {
                    const int wl = __ffsll((long long)nonzero) - 1;
                    nonzero &= nonzero - 1;
                    uint32_t m = __builtin_amdgcn_readlane(mine, wl);
                    const int base = (w0 + wl) << 5;
                    while (m) {
                        uint32_t r[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            // wave-uniform: the literal, its row, whether it is negated; unused slots read row 0 and give all ones
                            const bool used = m != 0;
                            const int lit = used ? base + __builtin_ctz(m) : 0;
                            m &= m - 1;
                            const bool negated = lit >= M;
                            const uint32_t flip = negated ? 0xFFFFFFFFu : 0u, fill = used ? 0u : 0xFFFFFFFFu;
                            r[u] = (col[(int64_t)(negated ? lit - M : lit) * row_words] ^ flip) | fill;
                        }
#pragma unroll
                        for (int u = 0; u < 8; ++u) acc &= r[u];
                    }
                }
            }
            if (MC > 64) {
                // more include words follow: the other waves need wave 0's row to decide the same way
                if (wave == 0 && active) handed[lane] = acc;
                __syncthreads();
                acc = active ? handed[lane] : 0u;
                __syncthreads();
            }
        }
        if (wave != 0) continue;
        for (int off = 32; off > 0; off >>= 1) included += __shfl_xor(included, off);
        const uint32_t v = active ? acc : 0u;
        if (lane == 0) n_incl[c] += included;
        fit_clause_tail(v, lane, words, NC, n_nodes, c, C, K, weights, k0, k1, step, finish != 0,
                        bitmap_out + (int64_t)c * NC, clause_node, class_sum, &partial);
    }
    if (wave == 0 && K <= 64 && lane < K && partial != 0) atomicAdd(&class_sum[lane], partial);
}
