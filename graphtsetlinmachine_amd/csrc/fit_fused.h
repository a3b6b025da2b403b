// One training step (tm.py:669-747) of a depth-1 model in two kernels.
//
//   k_fit_eval      K1 + K6 + K7: each wave takes clauses in turn.  The graph's
//                   literal-major rows (see score_tiles.h) are staged in LDS;
//                   the clause's truth over the graph's nodes is the AND of
//                   the rows of its included literals, read off the include
//                   plane of the automaton bank.  Writes the clause/node
//                   bitmap, the include count and the picked node, and adds
//                   the clause's weights to the class sums.
//   k_fit_feedback  K8 + K9: a block owns a few clauses; first one thread per
//                   (clause, class) decides the feedback and moves the weight,
//                   then one thread per (clause, automaton word) applies Type
//                   I / II feedback for the classes in order.
//
// Nothing but the class sums crosses clause boundaries, which is why the pair
// needs a single device-wide dependency per graph.
#pragma once

// Sum over the wave of a small per-lane count (< 64) from ballots of the count's bits: scalar
// population counts, no cross-lane data movement (a shuffle reduction is six dependent LDS-pipe
// round trips).
__device__ __forceinline__ int wave_sum_small(int count) {
    int t = 0;
#pragma unroll
    for (int bit = 0; bit < 6; ++bit) t += __popcll(__ballot((count >> bit) & 1)) << bit;
    return t;
}

constexpr int FIT_EVAL_BLOCK = 256;
constexpr int FIT_WALK_ALL = 40;      // clauses with at most this many literals AND all their rows (rows in global memory)
constexpr int FIT_WALK_ALL_LDS = 512; // the same with the rows staged in LDS
constexpr int FIT_FILTER_ROWS = 16;  // rows the others AND before testing nodes
constexpr int FIT_FEW_NODES = 2;    // up to this many surviving nodes (estimate) are tested one by one, more are filtered further
constexpr int FIT_QUEUE = 128;     // words of LDS per wave: included literals found in `order`, waiting for a batch of row reads

struct FitGraph {
    int tile;        // tile holding the graph
    int word0;       // first word of the graph's slot inside a tile row
    int words;       // words of the slot that hold nodes of this graph
    int shift;       // bit offset inside word0 (tiny graphs), else 0
    uint32_t mask;   // valid bits of the word (tiny graphs), else all ones
};

__host__ __device__ inline FitGraph fit_graph_slot(const TileGeom &tg, int graph, int n_nodes) {
    FitGraph f;
    f.tile = graph / tg.gpt;
    int j = graph - f.tile * tg.gpt;
    if (tg.slot_words > 0) {
        f.word0 = j * tg.slot_words;
        f.words = n_nodes == 0 ? 1 : (n_nodes - 1) / 32 + 1;
        f.shift = 0;
        f.mask = 0xFFFFFFFFu;
    } else {
        int bit = j * tg.slot_bits;
        f.word0 = bit >> 5;
        f.words = 1;
        f.shift = bit & 31;
        f.mask = tg.slot_bits >= 32 ? 0xFFFFFFFFu : ((1u << tg.slot_bits) - 1u);
    }
    return f;
}

// The end of a clause's evaluation for one graph, shared by every layer: lane L holds word L of
// the clause's truth over the graph's nodes.  Writes the clause's row of the clause/node bitmap
// and, when `finish` is set (the last layer), picks the node the clause learns from (K7,
// kernels.py:319-354) and adds the clause's weights to the class sums (K6, kernels.py:279-317;
// lanes k < K keep a running sum in *partial when K <= 64).
__device__ __forceinline__ void fit_clause_tail(uint32_t v, int lane, int words, int NC, int n_nodes, int c, int C, int K,
                                                const int32_t *__restrict__ weights, uint32_t k0, uint32_t k1,
                                                uint32_t step, bool finish, uint32_t *out,
                                                int32_t *__restrict__ clause_node, int32_t *class_sum, int *partial) {
    // chunks past the graph are left all ones, as kernels.py:443-466 leaves them
    for (int i = lane; i < NC; i += 64) out[i] = i < words ? (i == lane ? v : 0u) : 0xFFFFFFFFu;
    // the reference's arithmetic for a graph without nodes (kernels.py:289-295)
    if (n_nodes == 0 && lane == 0) out[0] = 0xFFFFFFFFu;
    if (!finish) return;
    // true nodes before this lane's word, and in total
    const int pc = __popc(v);
    int before = pc;
    for (int off = 1; off < 64; off <<= 1) {
        int t = __shfl_up(before, off);
        if (lane >= off) before += t;
    }
    const int true_nodes = __shfl(before, 63);
    before -= pc;
    bool fired = true_nodes > 0;
    int node = -1;
    if (n_nodes == 0) {
        fired = true;
    } else if (fired) {
        // K7: the pick-th true node, pick = (r * count) >> 32
        philox_out r = philox4x32_10((uint32_t)c, 0u, step, GTM_TAG_CLAUSE_NODE, k0, k1);
        const int pick = (int)(((uint64_t)r.v[0] * (uint64_t)true_nodes) >> 32);
        const bool mine = pick >= before && pick < before + pc;
        int candidate = 0;
        if (mine) {
            uint32_t t = v;
            for (int j = before; j < pick; ++j) t &= t - 1;
            candidate = lane * 32 + __ffs(t) - 1;
        }
        const unsigned long long owner = __ballot(mine);
        node = __shfl(candidate, __ffsll((long long)owner) - 1);
    }
    if (lane == 0) clause_node[c] = node;
    // K6
    if (fired) {
        if (K <= 64) {
            if (lane < K) *partial += weights[(int64_t)lane * C + c];
        } else {
            for (int k = lane; k < K; k += 64) atomicAdd(&class_sum[k], weights[(int64_t)k * C + c]);
        }
    }
}

// Truth of one clause over the nodes of a graph from literal-major rows: lane L of the wave gets the
// nodes of word L (`active` lanes hold a word of the graph; col = the lane's column of the rows, rows
// `stride` words apart).  inc = word 0 of the clause's include plane (words inc_stride apart).  A
// clause with more than `walk_all` literals ANDs the rows of its first FIT_FILTER_ROWS literals in
// `order` (the ones that hold least often in the data set) and then tests the few nodes that are
// left against its whole include mask on the nodes' own literal words (X_rows: the graph's
// node-major literal words, its first node's row).  Returns the lane's word of node bits (already
// shifted and masked for graphs that share a word); *included_out = the clause's literal count.
__device__ __forceinline__ uint32_t fit_clause_truth(const uint32_t *inc, int inc_stride, int LA, uint32_t filter,
                                                     const uint32_t *col, int stride, int literals, int type_row, int ones_row,
                                                     const FitGraph &fg, int n_nodes, int walk_all,
                                                     const uint32_t *__restrict__ X_rows, const uint32_t *__restrict__ order,
                                                     bool active, int lane, int *included_out, uint32_t *queue = nullptr) {
    // lane w fetches include word w0 + w: one memory latency for up to 64 words
    auto include_words = [&](int w0) {
        uint32_t mine = w0 + lane < LA ? inc[(int64_t)(w0 + lane) * inc_stride] : 0u;
        if (w0 + lane == LA - 1) mine &= filter;
        return mine;
    };
    int included = 0;
    uint32_t first_words = 0;
    for (int w0 = 0; w0 < LA; w0 += 64) {
        const uint32_t mine = include_words(w0);
        if (w0 == 0) first_words = mine;
        included += wave_sum_small(__popc(mine));
    }
    // A clause with many literals ANDs the rows of its first FIT_FILTER_ROWS only and then tests the
    // few nodes that are left against its whole include mask on the nodes' own literal words.
    const bool filter_only = included > walk_all && n_nodes > 0;
    uint32_t acc = active ? col[(int64_t)type_row * stride] : 0u;
    bool all_rows = false;  // every included literal's row has been applied: acc is the clause's truth
    if (filter_only && order) {
        // the first FIT_FILTER_ROWS included literals in `order` (the ones that hold least often in the
        // data set), 16 row reads in flight; while more than a few nodes survive, 16 more: one round
        // trip of row reads removes most of them, testing them costs a round trip per word of nodes.
        // A clause that still holds at many nodes after 32 rows is not one that a few rows decide:
        // it takes all its rows, and stops early only when no node is left.
        // With `queue` (FIT_QUEUE words of LDS of this wave's own) the included literals found in `order` wait
        // there until 16 are together: a clause of 70 of 2,048 literals finds two per 64 places of `order`, and a
        // batch of row reads per 64 places would be 32 memory round trips of 2 rows instead of 5 of 16.
        int budget = FIT_FILTER_ROWS, applied = 0;
        int r0 = 0;
        unsigned long long picked = 0ull;  // lanes whose literal (in `order`) is included and not applied yet
        uint32_t lit = 0u;
        int head = 0, tail = 0;  // with `queue`: its entries [head, tail), places counted modulo FIT_QUEUE
        for (;;) {
            if (budget <= 0) {
                const int mine = active ? __popc((acc >> fg.shift) & fg.mask) : 0;
                const int left = __popcll(__ballot(mine > 0)) + __popcll(__ballot(mine > 1));
                if (left <= FIT_FEW_NODES) break;
                budget = applied >= 32 ? 0x7FFFFFFF : 16;
            }
            int row[16];
            if (queue) {
                while (tail - head < 16 && r0 < literals) {
                    const int r = r0 + lane;
                    lit = r < literals ? order[r] : 0u;
                    uint32_t word = inc[(int64_t)(lit >> 5) * inc_stride];
                    if ((int)(lit >> 5) == LA - 1) word &= filter;
                    const bool mine = r < literals && ((word >> (lit & 31u)) & 1u);
                    picked = __ballot(mine);
                    if (mine) queue[(tail + __popcll(picked & ((1ull << lane) - 1ull))) & (FIT_QUEUE - 1)] = lit;
                    tail += __popcll(picked);
                    r0 += 64;
                }
                if (tail == head) {
                    all_rows = true;
                    break;
                }
                // (a wave's LDS accesses are carried out in order: the reads below see what was just written)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
                const int n = tail - head < 16 ? tail - head : 16;
#pragma unroll
                for (int u = 0; u < 16; ++u)
                    row[u] = u < n ? __builtin_amdgcn_readfirstlane((int)queue[(head + u) & (FIT_QUEUE - 1)]) : ones_row;
                head += n;
            } else {
                if (picked == 0ull) {
                    if (r0 >= literals) {
                        all_rows = true;
                        break;
                    }
                    const int r = r0 + lane;
                    lit = r < literals ? order[r] : 0u;
                    uint32_t word = inc[(int64_t)(lit >> 5) * inc_stride];
                    if ((int)(lit >> 5) == LA - 1) word &= filter;
                    picked = __ballot(r < literals && ((word >> (lit & 31u)) & 1u));
                    r0 += 64;
                    continue;
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    row[u] = picked ? (int)__builtin_amdgcn_readlane(lit, __ffsll((long long)picked) - 1) : ones_row;
                    picked &= picked - 1;
                }
            }
            uint32_t r16[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) r16[u] = col[(int64_t)row[u] * stride];
#pragma unroll
            for (int u = 0; u < 16; ++u) acc &= r16[u];
            budget -= 16, applied += 16;
            if (applied > 32 && __ballot(acc != 0u) == 0ull) {  // (all the rows are wanted, but no node is left)
                all_rows = true;
                break;
            }
        }
    } else {
        // The literals in the order of the include words, 16 rows per batch of reads whatever words they come from (a
        // clause of 30 literals has them in 25 of its 64 words: a batch per word would be 25 memory round trips of
        // one or two rows).  Scalar state: the word at hand, what is left of it, the words still to come.
        int budget = filter_only ? FIT_FILTER_ROWS : 0x7FFFFFFF;
        for (int w0 = 0; w0 < LA && budget > 0; w0 += 64) {
            const uint32_t mine = w0 == 0 ? first_words : include_words(w0);
            unsigned long long nonzero = __ballot(mine != 0);
            uint32_t m = 0u;
            int base = 0;
            auto next_word = [&]() {  // on to the next word that holds literals; false: none is left
                if (!nonzero) return false;
                const int wl = __ffsll((long long)nonzero) - 1;
                nonzero &= nonzero - 1;
                m = __builtin_amdgcn_readlane(mine, wl);
                base = (w0 + wl) << 5;
                return true;
            };
            bool more = next_word();
            while (more && budget > 0) {
                int row[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const bool used = more;
                    row[u] = used ? base + __builtin_ctz(m) : ones_row;
                    if (used) {
                        m &= m - 1;
                        if (m == 0u) more = next_word();
                    }
                }
                uint32_t r[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) r[u] = col[(int64_t)row[u] * stride];
#pragma unroll
                for (int u = 0; u < 16; ++u) acc &= r[u];
                budget -= 16;
            }
        }
    }
    uint32_t v = active ? (acc >> fg.shift) & fg.mask : 0u;
    if (filter_only && !all_rows) {
        // Lane L holds nodes 32 L .. 32 L + 31.  The surviving nodes are walked on the scalar unit, 8 at
        // a time; for each, lane w compares include word w with the node's literal word w (one
        // coalesced load per node and 64 words), and a node with any violated word is cleared.
        unsigned long long live = __ballot(v != 0);
        while (live) {
            const int L = __ffsll((long long)live) - 1;
            live &= live - 1;
            uint32_t word = __builtin_amdgcn_readlane(v, L);
            uint32_t cleared = 0;
            while (word) {
                int bit[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    bit[u] = word ? __builtin_ctz(word) : -1;
                    word &= word - 1;
                }
                uint32_t violated[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int w0 = 0; w0 < LA; w0 += 64) {
                    const uint32_t mine = w0 == 0 ? first_words : include_words(w0);
                    const bool in_row = w0 + lane < LA;
                    uint32_t xs[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        xs[u] = in_row ? X_rows[(int64_t)(L * 32 + (bit[u] < 0 ? 0 : bit[u])) * LA + w0 + lane] : 0xFFFFFFFFu;
#pragma unroll
                    for (int u = 0; u < 8; ++u) violated[u] |= mine & ~xs[u];
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (bit[u] >= 0 && __ballot(violated[u] != 0) != 0) cleared |= 1u << bit[u];
            }
            if (lane == L) v &= ~cleared;
        }
    }
    *included_out = included;
    return v;
}

// K1 + K6 + K7 for one graph.  A block stages the graph's literal-major rows
// (plus an all-ones row) in LDS; each wave then takes clauses in turn.  The
// clause is wave-uniform: its include words come in by scalar loads straight
// from the top bit plane of the automaton bank, their set bits are walked on
// the scalar unit, and lane L ANDs word L of every included literal's row, 8
// LDS reads in flight at a time.  STAGE = false reads the rows from the tile
// in global memory instead (graphs whose rows do not fit in LDS).  `finish` = 0
// (models with message layers) stops after the bitmap and the include counts.
// X_rows: the graph's node-major literal words (its first node's row); order:
// the literals sorted by how often they hold in the data set, rarest first.
template <bool STAGE>
__global__ __launch_bounds__(FIT_EVAL_BLOCK) void k_fit_eval(
    const uint32_t *__restrict__ tiles, TileGeom tg, FitGraph fg, int n_nodes, int literals, int n_types, int C, int LA,
    int B, int K, int NC, uint32_t filter, const uint32_t *__restrict__ bank, const int32_t *__restrict__ weights,
    uint32_t k0, uint32_t k1, uint32_t step, int finish, const uint32_t *__restrict__ X_rows,
    const uint32_t *__restrict__ order, uint32_t *__restrict__ bitmap, int32_t *__restrict__ n_incl, int32_t *__restrict__ clause_node,
    int32_t *class_sum) {
    extern __shared__ uint32_t rows_lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int WAVES = FIT_EVAL_BLOCK / 64;
    const uint32_t *tile = tiles + (int64_t)fg.tile * tg.rows * tg.tw + fg.word0;
    const int stride = STAGE ? fg.words : tg.tw;
    const int ones_row = literals + n_types;  // in the tile this is the all-ones row as well
    const uint32_t *rows = tile;
    if (STAGE) {
        const int total = (literals + n_types + 1) * fg.words;
        for (int base = 0; base < total; base += FIT_EVAL_BLOCK * 8) {
            uint32_t v[8];
            int at[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                int i = base + u * FIT_EVAL_BLOCK + tid;
                int r = i / fg.words, w = i - r * fg.words;
                at[u] = i < total ? i : -1;
                v[u] = i < total ? tile[(int64_t)r * tg.tw + w] : 0u;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (at[u] >= 0) rows_lds[at[u]] = v[u];
        }
        __syncthreads();
        rows = rows_lds;
    }

    const bool active = lane < fg.words;
    const uint32_t *col = rows + (active ? lane : 0);
    __shared__ uint32_t queue_of_wave[WAVES][FIT_QUEUE];
    int partial = 0;  // lane k < K: this wave's contribution to class k
    for (int c = blockIdx.x * WAVES + wave; c < C; c += gridDim.x * WAVES) {
        int included;
        const uint32_t v = fit_clause_truth(bank + (int64_t)c * LA * B + (B - 1), B, LA, filter, col, stride, literals,
                                            literals + c % n_types, ones_row, fg, n_nodes,
                                            STAGE ? FIT_WALK_ALL_LDS : FIT_WALK_ALL, X_rows, order, active, lane, &included,
                                            queue_of_wave[wave]);
        if (lane == 0) n_incl[c] = included;
        fit_clause_tail(v, lane, fg.words, NC, n_nodes, c, C, K, weights, k0, k1, step, finish != 0,
                        bitmap + (int64_t)c * NC, clause_node, class_sum, &partial);
    }
    if (K <= 64 && lane < K && partial != 0) atomicAdd(&class_sum[lane], partial);
}

// kernels.py:55-96 on one word of 32 automata whose MAXB >= B bit planes sit in registers.
template <int MAXB>
__device__ __forceinline__ void reg_inc(uint32_t (&ta)[MAXB], int B, uint32_t active) {
    uint32_t carry = active;
#pragma unroll
    for (int b = 0; b < MAXB; ++b)
        if (b < B) {
            uint32_t v = ta[b];
            ta[b] = v ^ carry;
            carry &= v;
        }
#pragma unroll
    for (int b = 0; b < MAXB; ++b)
        if (b < B) ta[b] |= carry;  // residual carry: saturate
}

template <int MAXB>
__device__ __forceinline__ void reg_dec(uint32_t (&ta)[MAXB], int B, uint32_t active) {
    uint32_t carry = active;
#pragma unroll
    for (int b = 0; b < MAXB; ++b)
        if (b < B) {
            uint32_t v = ta[b];
            ta[b] = v ^ carry;
            carry &= ~v;
        }
#pragma unroll
    for (int b = 0; b < MAXB; ++b)
        if (b < B) ta[b] &= ~carry;
}

// Type I / II feedback of kernels.py:141-183 (and :98-139 for message banks)
// for all classes in order on one automaton word; returns the include plane.
// `fb_of`, when not NULL, holds the feedback bits of class k at fb_of[k] (computed elsewhere by the
// same gtm_feedback_bits call).
template <int MAXB>
__device__ __forceinline__ uint32_t feedback_word(uint32_t *ta_global, int B, int K, const int32_t *u_of, int u_stride,
                                                  bool fired, bool within, int boost, uint32_t x, uint32_t k0,
                                                  uint32_t k1, uint32_t c, uint32_t w, uint32_t step, uint32_t bank_id,
                                                  uint32_t thr16, const uint32_t *fb_of = nullptr) {
    uint32_t ta[MAXB];
    // 8 planes (the default): the word's planes are 32 contiguous, 32-byte aligned bytes
    const bool vector8 = MAXB == 8 && B == 8 && (reinterpret_cast<uintptr_t>(ta_global) & 31u) == 0;
    if (vector8) {
        const uint4 lo = reinterpret_cast<const uint4 *>(ta_global)[0], hi = reinterpret_cast<const uint4 *>(ta_global)[1];
        ta[0] = lo.x, ta[1] = lo.y, ta[2] = lo.z, ta[3] = lo.w;
        if (MAXB >= 8) ta[4 % MAXB] = hi.x, ta[5 % MAXB] = hi.y, ta[6 % MAXB] = hi.z, ta[7 % MAXB] = hi.w;
    } else {
#pragma unroll
        for (int b = 0; b < MAXB; ++b) ta[b] = b < B ? ta_global[b] : 0u;
    }
    for (int k = 0; k < K; ++k) {
        const int u = u_of[(int64_t)k * u_stride];
        if (u > 0) {
            uint32_t fb = fb_of ? fb_of[k] : gtm_feedback_bits(k0, k1, c, w, step, bank_id, (uint32_t)k, thr16);
            if (fired && within) {
                reg_inc<MAXB>(ta, B, boost == 1 ? x : (x & ~fb));
                reg_dec<MAXB>(ta, B, ~x & fb);
            } else {
                reg_dec<MAXB>(ta, B, fb);
            }
        } else if (u < 0 && fired) {
            uint32_t top = 0;
#pragma unroll
            for (int b = 0; b < MAXB; ++b)
                if (b == B - 1) top = ta[b];
            reg_inc<MAXB>(ta, B, ~x & ~top);
        }
    }
    uint32_t top = 0;
    if (vector8) {
        reinterpret_cast<uint4 *>(ta_global)[0] = make_uint4(ta[0], ta[1], ta[2], ta[3]);
        reinterpret_cast<uint4 *>(ta_global)[1] = make_uint4(ta[4 % MAXB], ta[5 % MAXB], ta[6 % MAXB], ta[7 % MAXB]);
        return ta[7 % MAXB];
    }
#pragma unroll
    for (int b = 0; b < MAXB; ++b)
        if (b < B) {
            ta_global[b] = ta[b];
            if (b == B - 1) top = ta[b];
        }
    return top;
}

__device__ __forceinline__ uint32_t feedback_word_any(uint32_t *ta_global, int B, int K, const int32_t *u_of,
                                                      int u_stride, bool fired, bool within, int boost, uint32_t x,
                                                      uint32_t k0, uint32_t k1, uint32_t c, uint32_t w, uint32_t step,
                                                      uint32_t bank_id, uint32_t thr16, const uint32_t *fb_of = nullptr) {
    if (B <= 8)
        return feedback_word<8>(ta_global, B, K, u_of, u_stride, fired, within, boost, x, k0, k1, c, w, step, bank_id, thr16, fb_of);
    if (B <= 16)
        return feedback_word<16>(ta_global, B, K, u_of, u_stride, fired, within, boost, x, k0, k1, c, w, step, bank_id, thr16, fb_of);
    return feedback_word<32>(ta_global, B, K, u_of, u_stride, fired, within, boost, x, k0, k1, c, w, step, bank_id, thr16, fb_of);
}

// Sum over the wave of a small per-lane count (< 64), and the sum over the lanes below this one,
// from ballots of the count's bits: no cross-lane data movement.
__device__ __forceinline__ void wave_count_scan(int count, int lane, int *total, int *before) {
    const unsigned long long below = (1ull << lane) - 1ull;
    int t = 0, b = 0;
#pragma unroll
    for (int bit = 0; bit < 6; ++bit) {
        const unsigned long long has = __ballot((count >> bit) & 1);
        t += __popcll(has) << bit;
        b += __popcll(has & below) << bit;
    }
    *total = t;
    *before = b;
}

// The automaton banks one training step updates: bank 0 holds the literals of
// the nodes (rows = the graph's X rows), bank l > 0 the message literals of
// layer l (rows = that layer's messages, one row of `chunks` words per node).
struct FitBanks {
    int n;
    int total_chunks;  // sum of chunks[]
    uint32_t *bank[GTM_MAX_DEPTH];
    const uint32_t *rows[GTM_MAX_DEPTH];
    int chunks[GTM_MAX_DEPTH];
    uint32_t thr16[GTM_MAX_DEPTH];
};

// K8 + K9 (+ K10 for the message banks) for `cpb` clauses per block; see the header comment.
__global__ void k_fit_feedback(FitBanks banks, int32_t *weights, const int32_t *class_sum,
                               int32_t *class_sum_next, const int32_t *__restrict__ y, int C, int B, int K,
                               int T, int negative, int boost, int max_included, uint64_t q_thr,
                               uint32_t k0, uint32_t k1, uint32_t step,
                               const int32_t *__restrict__ clause_node, const int32_t *__restrict__ n_incl, int cpb) {
    extern __shared__ int32_t upd[];  // [cpb][K]
    const int tid = threadIdx.x;
    const int c_base = blockIdx.x * cpb;
    if (blockIdx.x == 0)  // the next step accumulates into the other buffer
        for (int k = tid; k < K; k += blockDim.x) class_sum_next[k] = 0;

    for (int i = tid; i < cpb * K; i += blockDim.x) {
        const int c = c_base + i / K, k = i % K;
        int u = 0;
        if (c < C) {
            int cs = class_sum[k];
            cs = cs > T ? T : (cs < -T ? -T : cs);
            const int yk = y[k];
            const int target = 1 - 2 * (cs > yk);
            int w = weights[(int64_t)k * C + c];
            const int sign = (w >= 0) - (w < 0);
            int err = yk - cs;
            err = err < 0 ? -err : err;
            philox_out r = philox4x32_10((uint32_t)c, (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, k0, k1);
            const bool skip = (target == -1 && (uint64_t)r.v[0] >= q_thr) ||
                              ((uint64_t)r.v[1] * (uint64_t)(2 * (int64_t)T) >= ((uint64_t)err << 32));
            u = skip ? 0 : target * sign;
            const bool fired = clause_node[c] != -1;
            if (u > 0 && fired && (w < 0 ? -(int64_t)w : (int64_t)w) < 2147483647) {
                weights[(int64_t)k * C + c] = w + sign;
            } else if (u < 0 && fired) {
                w -= sign;
                if (negative == 0 && w < 1) w = 1;
                weights[(int64_t)k * C + c] = w;
            }
        }
        upd[i] = u;
    }
    __syncthreads();

    const int per_clause = banks.total_chunks;
    for (int i = tid; i < cpb * per_clause; i += blockDim.x) {
        const int local = i / per_clause;
        int w = i - local * per_clause;
        const int c = c_base + local;
        if (c >= C) continue;
        const int32_t *u_of = upd + local * K;
        bool any = false;
        for (int k = 0; k < K; ++k) any |= u_of[k] != 0;
        if (!any) continue;
        // which bank the word belongs to (static indices: the struct stays in scalar registers)
        int l = 0, chunks = banks.chunks[0], first = 0;
        uint32_t *bank = banks.bank[0];
        const uint32_t *rows = banks.rows[0];
        uint32_t thr16 = banks.thr16[0];
        int start = banks.chunks[0];
#pragma unroll
        for (int t = 1; t < GTM_MAX_DEPTH; ++t) {
            if (t < banks.n && w >= start) {
                l = t;
                first = start;
                chunks = banks.chunks[t];
                bank = banks.bank[t];
                rows = banks.rows[t];
                thr16 = banks.thr16[t];
            }
            start += t < banks.n ? banks.chunks[t] : 0;
        }
        w -= first;
        const int node = clause_node[c];
        const bool fired = node != -1;
        const bool within = n_incl[c] <= max_included;
        const uint32_t x = fired ? rows[(int64_t)node * chunks + w] : 0u;
        uint32_t *ta = bank + ((int64_t)c * chunks + w) * B;
        feedback_word_any(ta, B, K, u_of, 1, fired, within, boost, x, k0, k1, (uint32_t)c, (uint32_t)w, step,
                          (uint32_t)l, thr16);
    }
}
