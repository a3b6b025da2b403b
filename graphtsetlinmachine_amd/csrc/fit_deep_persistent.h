// A whole run of training examples (the loop at tm.py:669-747) of a model WITH
// message layers in ONE cooperative launch.
//
// As in fit_persistent.h every workgroup owns a contiguous range of clauses for
// the whole run and keeps their automata - all banks, all bit planes - and
// weights in LDS.  What crosses clause boundaries per example is, per message
// layer, what the nodes receive (kernels.py:549-590) and, at the end, the class
// sums (kernels.py:310-315).  Per example and message layer:
//
//   a. every workgroup sends what its own clauses contribute, literal-major: for a
//      clause that is true at the nodes S it first collects in LDS, per edge type t,
//      the row of nodes that some node of S points at with an edge of type t, and
//      then ORs that row into row (h + t) mod M of what the nodes RECEIVE, for every
//      bit h of the clause's hypervector (kernels.py:581: a message bit travels along
//      an edge shifted by the edge's type) - device-scope atomic OR, only words that
//      hold a node;
//   -- one device-wide wait: every contribution is in --
//   b. every workgroup copies all M received rows into LDS and evaluates its
//      clauses on them: truth AND the rows of the included message literals,
//      complemented for the negated ones (kernels.py:505-527), the automaton words of
//      a clause spread over the workgroup's waves.
//
// After the last layer: node pick (K7), votes, the class-sum exchange of
// fit_persistent.h (sums and arrival count in one 64-bit word per class), the
// feedback decisions (K8) and Type I / II feedback on every bank (K9, K10) with the
// literal words of the picked node - its X row for bank 0, bit `node` of the
// received rows of layer l for bank l.
//
// Nothing is exchanged through ordinary stores and no cache is flushed: every
// word another workgroup reads is written with a device-scope atomic (carried out
// where all workgroups see it) that the writer waits for - its wave's count of
// outstanding memory operations falls to zero - before it announces its arrival,
// and read with a device-scope atomic load after the reader has seen every arrival.  The
// received rows live in a ring of three slots (example i uses slot i mod 3).  A
// workgroup clears its share of slot (i + 1) mod 3 during example i: whoever is in
// example i has seen every workgroup arrive at the class sums of example i - 1, so
// nobody reads that slot's last contents (example i - 2) any more, and the first
// contribution of example i + 1 cannot precede this workgroup's arrival at the
// class sums of example i, which it makes after the clearing.  Arrival counters
// only ever grow.
//
// Two layouts (template flag BIG).  Small models keep the automata of the own clauses in LDS, next to
// the layer-0 rows of the graph and all M received rows.  Where that does not fit (8000 clauses on
// 841-node graphs with 2048 literals), the automata stay in global memory - a workgroup only ever
// touches those of its own clauses, with ordinary loads and stores - and LDS holds a copy of their
// include planes; layer 0 reads the literal rows it needs from the tiles in place; the received rows
// pass through LDS a window of rows at a time; and what each node received is also published
// node-major (`vec`: every workgroup turns the bits of its share of the nodes while a window is in
// LDS), so that the message literals of a picked node are words to load, not bits to collect.
//
// Every wait is bounded (`spin_limit` polls); a workgroup that gives up raises the
// abort flag and every workgroup leaves at its next wait, so the grid always drains.
#pragma once

#ifdef FITD_CLOCKS  // development aid: workgroup 0 adds up the time between its phases (100 MHz ticks)
#define FITD_TICK(k)                                                   \
    if (g == 0 && tid == 0) {                                          \
        const unsigned long long now_ = wall_clock64();                \
        clk[k] += now_ - last_;                                        \
        last_ = now_;                                                  \
    }
#else
#define FITD_TICK(k)
#endif

constexpr int FITD_BLOCK = 1024;
// An arrival counter is kept as this many partial words, one per lane of the wave that adds them up: adds to
// one word are carried out one after the other (about 30 ns each measured), and 200 workgroups arrive at once.
constexpr int FITD_PARTS = 64;
constexpr int FITD_STRIDE = 16;       // 64-bit words between two of them: a cache line each
constexpr int FITD_MAX_EDGE_TYPES = 16;

struct FitDeepParams {
    // data set
    const uint32_t *tiles, *X, *node_index, *n_nodes, *n_edges, *edge_index, *edge;
    const uint32_t *order;  // the literals, the ones that hold least often in the data set first
    const int32_t *encoded_Y;
    TileGeom tg;
    int first_example, n_examples;
    uint32_t first_step;
    // model
    uint32_t *bank[GTM_MAX_DEPTH];
    int32_t *weights;
    const uint32_t *hv;
    int depth, literals, n_types, C, LA, MC, MW, M, MB, B, K, T, negative, boost, max_included, has_edges;
    uint32_t filter, thr16[GTM_MAX_DEPTH], k0, k1;
    uint64_t q_thr;
    // exchange (device memory, zero on entry)
    uint32_t *got;                  // [3][depth - 1][M][NW]
    uint32_t *vec;                  // [depth - 1][max_nodes][MW] what each node received, node-major (BIG only)
    unsigned long long *arrived;    // [depth - 1][FITD_PARTS * FITD_STRIDE]
    unsigned long long *class_sum;  // [3][K][FITP_SUM_PARTS] words FITP_SUM_STRIDE apart
    uint32_t *abort_flag;
    uint32_t spin_limit;
    unsigned long long wait_ticks;
    int force_abort;
    int clauses_per_group;
    const int *perm;  // [groups][clauses_per_group] the clause in each workgroup's slots, -1 after its last; NULL: clauses in order
    int NW;          // words of a row over the nodes of the largest graph
    int rows_words;  // LDS words of the staged layer-0 rows: (literals + n_types + 1) * NW; 0 when they are read in place (BIG)
    int window_rows; // received rows that pass through LDS at a time: a multiple of 32, M unless BIG
    int by_masks;    // phase a goes over the edges once for 32 clauses (the window's LDS is large enough for that)
    int max_nodes;   // nodes of the largest graph
    int edge_cap;    // edges of the graph that has most (0 without edges)
    int edge_types;  // largest edge type + 1 (at most FITD_MAX_EDGE_TYPES)
#ifdef FITD_CLOCKS
    unsigned long long *clocks;
#endif
};

// LDS words of the kernel.  big: rows_words == 0 and window_rows <= M; else window_rows == M.
inline size_t fit_deep_lds_words(bool big, int depth, int literals, int per_group, int LA, int MC, int MB, int B, int K, int NW, int rows_words,
                                 int window_rows, int max_nodes, int edge_cap, int edge_types) {
    const size_t per_clause = (size_t)LA + (size_t)(depth - 1) * MC;
    return 2 * ((size_t)rows_words + 2 * (size_t)max_nodes + (size_t)edge_cap + (size_t)K) + (size_t)window_rows * NW +
           (size_t)per_group * edge_types * NW + (size_t)per_group * per_clause * (big ? 1 : B) + 2 * (size_t)per_group * K +
           2 * (size_t)per_group + (size_t)per_group * NW + 2 * (size_t)K + 6 * (size_t)K +
           (big ? (size_t)literals : (size_t)per_group * (depth - 1) * MC) + (size_t)per_group * MB + (size_t)per_group +
           (big ? (size_t)(FITD_BLOCK / 64) * FIT_QUEUE : 0) + 64;
}

// What the cooperative kernel has to know about the edges of a run of examples: [0] most edges of
// one graph, [1] largest edge type, [2] != 0 when some graph's edges are not stored node after node
// (edge_index[n + 1] == edge_index[n] + number_of_graph_node_edges[n]) or point outside the graph.
// One workgroup per example.
__global__ void k_edge_limits(const uint32_t *__restrict__ n_nodes, const uint32_t *__restrict__ node_index,
                              const uint32_t *__restrict__ n_edges, const uint32_t *__restrict__ edge_index,
                              const uint32_t *__restrict__ edge, int first_example, uint32_t *out) {
    const int ex = first_example + (int)blockIdx.x;
    const int n = (int)n_nodes[ex];
    if (n == 0) return;
    const int64_t base = node_index[ex];
    const uint32_t e0 = edge_index[base];
    const uint32_t total = edge_index[base + n - 1] + n_edges[base + n - 1] - e0;
    uint32_t irregular = 0u, top = 0u;
    for (int j = threadIdx.x; j < n - 1; j += blockDim.x)
        irregular |= edge_index[base + j + 1] != edge_index[base + j] + n_edges[base + j];
    for (uint32_t e = threadIdx.x; e < total && total < (1u << 24); e += blockDim.x) {
        irregular |= edge[(int64_t)(e0 + e) * 2] >= (uint32_t)n;
        top = max(top, edge[(int64_t)(e0 + e) * 2 + 1]);
    }
    if (threadIdx.x == 0) atomicMax(&out[0], total);
    if (top) atomicMax(&out[1], top);
    if (irregular) atomicOr(&out[2], 1u);
}

__device__ __forceinline__ uint32_t fitd_load(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wave 0 of a workgroup waits until the counter (the sum of its parts) has reached `target`.
__device__ __forceinline__ bool fitd_wait(const unsigned long long *parts, unsigned long long target,
                                          uint32_t *abort_flag, uint32_t spin_limit, unsigned long long wait_ticks,
                                          int force_abort, int lane) {
    if (force_abort) {
        __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    uint32_t polls = 0;
    unsigned long long waiting_since = 0ull;
    for (;;) {
        unsigned long long v = lane < FITD_PARTS
                                   ? __hip_atomic_load(&parts[lane * FITD_STRIDE], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                   : 0ull;
#pragma unroll
        for (int off = 1; off < FITD_PARTS; off <<= 1) v += __shfl_xor(v, off);
        v = __shfl(v, 0);
        if (v >= target) return true;
        if (__hip_atomic_load(abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 ||
            fit_wait_is_over(polls, spin_limit, waiting_since, wait_ticks)) {
            __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

// A 32 x 32 bit matrix held one row per lane (both halves of a wave hold one each): afterwards lane b
// holds column b, i.e. bit k of its word = bit b of what lane k (of the same half) held.
// (the form with a choice per lane instead of tile_transpose32's per-lane constants: this kernel has no vector
// registers to spare for them)
template <int J, uint32_t M>
__device__ __forceinline__ uint32_t fitd_transpose_step(uint32_t v, int lane) {
    const uint32_t p = tile_lane_xor<J>(v, lane);
    return (lane & J) ? ((p >> J) & M) | (v & ~M) : (v & M) | ((p & M) << J);
}
__device__ __forceinline__ uint32_t fitd_transpose32(uint32_t a, int lane) {
    a = fitd_transpose_step<16, 0x0000FFFFu>(a, lane);
    a = fitd_transpose_step<8, 0x00FF00FFu>(a, lane);
    a = fitd_transpose_step<4, 0x0F0F0F0Fu>(a, lane);
    a = fitd_transpose_step<2, 0x33333333u>(a, lane);
    return fitd_transpose_step<1, 0x55555555u>(a, lane);
}

// acc &= the rows of the literals that words [w_lo, w_hi) of an include plane hold - and, with `twin` >= 0,
// words [twin + w_lo, twin + w_hi) as well, in the same pass (the negated halves of a message bank's words; at
// most 32 words then) - and adds how many they hold to *included (an LDS counter).  `inc` points at the include
// plane's word 0 (words inc_stride apart); row r of the literal rows is at col[(r - row_base) * stride] for this
// lane; literals >= `half` are negated: the complement of row (literal - half) when `complement`, else a row of
// their own.  One wave.  PACKED: a batch of row reads takes literals from as many include words as it needs (for
// clauses whose include words hold one or two literals each); else a word's literals, eight at a time.
template <bool PACKED, typename Rows>
__device__ __forceinline__ void fitd_and_rows(const uint32_t *inc, int inc_stride, int w_lo, int w_hi, int twin, int last_word,
                                              uint32_t filter, Rows col, int stride, int row_base, int half, bool complement,
                                              int ones_row, uint32_t &acc, int *included, int lane) {
    const int span = twin >= 0 ? w_hi - w_lo : 64;  // lanes [0, span): the words themselves; [span, 2 span): their twins
    for (int w0 = w_lo; w0 < w_hi; w0 += 64) {
        const int mine_is = lane < span ? w0 + lane : twin + w0 + lane - span;  // the include word this lane holds
        const bool holds = lane < span ? w0 + lane < w_hi : lane < 2 * span;
        uint32_t mine = holds ? inc[mine_is * inc_stride] : 0u;
        if (mine_is == last_word) mine &= filter;
        if (mine != 0u) atomicAdd(included, __popc(mine));
        unsigned long long nonzero = __ballot(mine != 0);
        if constexpr (PACKED) {
            // The set bits of the held words, word after word, eight rows per batch of reads whatever words they
            // come from: with a batch per word, a clause of a hundred literals in 64 words read eight rows for every
            // one or two that it wanted.  (All of this is the same for every lane: scalar state.)
            uint32_t m = 0u, flip = 0u;
            int row0 = 0;
            auto next_word = [&]() {  // on to the next word that holds literals; false: none is left
                if (!nonzero) return false;
                const int wl = __ffsll((long long)nonzero) - 1;
                nonzero &= nonzero - 1;
                m = __builtin_amdgcn_readlane(mine, wl);
                const int first = (wl < span ? w0 + wl : twin + w0 + wl - span) << 5;
                const bool negated = complement && first >= half;  // (a word holds positive or negated literals, never both)
                row0 = (negated ? first - half : first) - row_base;
                flip = negated ? 0xFFFFFFFFu : 0u;
                return true;
            };
            bool more = next_word();
            while (more) {
                if (__ballot(acc != 0u) == 0ull) break;  // false everywhere stays false: only the count matters
                uint32_t r[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const bool used = more;
                    const int row = used ? row0 + __builtin_ctz(m) : ones_row - row_base;
                    r[u] = (col[(int64_t)row * stride] ^ (used ? flip : 0u)) | (used ? 0u : 0xFFFFFFFFu);
                    if (used) {
                        m &= m - 1;
                        if (m == 0u) more = next_word();
                    }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) acc &= r[u];
            }
        } else {
            while (nonzero) {
                if (__ballot(acc != 0u) == 0ull) break;  // false everywhere stays false: only the count matters
                const int wl = __ffsll((long long)nonzero) - 1;
                nonzero &= nonzero - 1;
                uint32_t m = __builtin_amdgcn_readlane(mine, wl);
                const int first = (wl < span ? w0 + wl : twin + w0 + wl - span) << 5;
                const bool negated = complement && first >= half;  // (a word holds positive or negated literals, never both)
                const int row0 = (negated ? first - half : first) - row_base;
                const uint32_t flip = negated ? 0xFFFFFFFFu : 0u;
                while (m) {
                    uint32_t r[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const bool used = m != 0;
                        const int row = used ? row0 + __builtin_ctz(m) : ones_row - row_base;
                        m &= m - 1;
                        r[u] = (col[(int64_t)row * stride] ^ flip) | (used ? 0u : 0xFFFFFFFFu);
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc &= r[u];
                }
            }
        }
    }
}

// Clauses dealt out to the workgroups by what they cost.  A workgroup owns its clauses for a whole launch, and
// an example takes as long as the slowest workgroup: with clauses in order, 32 to a workgroup, the sum of 32
// costs that differ by an order of magnitude (a clause of a hundred literals that holds at many nodes walks all
// its rows; an empty one costs next to nothing) varies by a third between workgroups.  Between launches of a
// run of examples the clauses are therefore sorted by the number of literals they include in all banks - what
// a clause's evaluation and feedback walk - and dealt out in rounds, back and forth over the workgroups, so
// that every workgroup gets the same mix.  Nothing moves: the table says which clause sits in which slot.
constexpr int FITD_DEAL_MAX = 8192;    // clauses that one workgroup sorts in LDS

struct FitDeepBanks {
    const uint32_t *bank[GTM_MAX_DEPTH];
};

// cost[c] = included literals of clause c over all banks (one wave per clause)
__global__ void k_fit_deep_cost(FitDeepBanks banks, int depth, int C, int LA, int MC, int B, uint32_t *__restrict__ cost) {
    const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (c >= C) return;
    uint32_t n = 0u;
    for (int l = 0; l < depth; ++l) {
        const int chunks = l == 0 ? LA : MC;
        for (int w = lane; w < chunks; w += 64) n += (uint32_t)__popc(banks.bank[l][((int64_t)c * chunks + w) * B + (B - 1)]);
    }
    for (int off = 32; off > 0; off >>= 1) n += __shfl_xor(n, off);
    if (lane == 0) cost[c] = n;
}

// One workgroup of 1,024 threads: the clauses sorted by cost, dearest first (ties by clause number), and dealt
// out: the clause at place r * G + j goes to slot r of workgroup j (r even) or G - 1 - j (r odd).  Dynamic LDS:
// 8 bytes per clause, rounded up to a power of two.
__global__ __launch_bounds__(1024) void k_fit_deep_deal(const uint32_t *__restrict__ cost, int C, int G, int own_max,
                                                         int *__restrict__ perm) {
    extern __shared__ unsigned long long deal_keys[];
    int N = 1;
    while (N < C) N <<= 1;
    for (int i = threadIdx.x; i < N; i += 1024)  // descending by cost, then ascending by clause: ~clause in the low word
        deal_keys[i] = i < C ? ((unsigned long long)cost[i] << 32) | (uint32_t)(0x7FFFFFFF - i) : 0ull;
    for (int i = threadIdx.x; i < G * own_max; i += 1024) perm[i] = -1;
    __syncthreads();
    for (int k = 2; k <= N; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < N; i += 1024) {
                const int partner = i ^ j;
                if (partner > i) {
                    const unsigned long long a = deal_keys[i], b = deal_keys[partner];
                    const bool descending = (i & k) == 0;
                    if (descending ? a < b : a > b) deal_keys[i] = b, deal_keys[partner] = a;
                }
            }
            __syncthreads();
        }
    for (int at = threadIdx.x; at < C; at += 1024) {
        const int c = 0x7FFFFFFF - (int)(uint32_t)deal_keys[at];
        const int r = at / G, j = at - r * G;
        perm[((r & 1) ? G - 1 - j : j) * own_max + r] = c;
    }
}

// MAXB: bit planes of an automaton kept in registers while a word is updated (>= B).
// BIG: automata in global memory, layer-0 rows read in place, received rows in windows (see the top).
template <int MAXB, bool BIG>
__global__ __launch_bounds__(FITD_BLOCK) void k_fit_deep_persistent(FitDeepParams p) {
    extern __shared__ uint32_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int WAVES = FITD_BLOCK / 64;
    const int G = (int)gridDim.x, g = (int)blockIdx.x;
    const int own_max = p.clauses_per_group;
    const int LA = p.LA, MC = p.MC, MW = p.MW, M = p.M, B = p.B, K = p.K, NW = p.NW, L = p.depth - 1, TE = p.edge_types;
    const int WR = p.window_rows;
    const int per_clause = LA + L * MC;  // automaton words of a clause over all banks
    const int SB = BIG ? 1 : B;          // LDS words per automaton word: the include plane, or every plane

    // LDS carve-up
    // per example, twice (the next example's are fetched while this one waits):
    //   [rows_words] staged layer-0 rows of the graph, [max_nodes] first edge of a node counted from the
    //   graph's first, [max_nodes] edges of a node, [edge_cap] destination | type << 16, [K] encoded labels
    const size_t staged_words = (size_t)p.rows_words + 2 * (size_t)p.max_nodes + (size_t)p.edge_cap + (size_t)K;
    uint32_t *mrows = lds + 2 * staged_words;                     // [WR][NW] received rows of the current layer (a window of them)
    uint32_t *reach = mrows + (size_t)WR * NW;                    // [own][TE][NW] nodes reached from a clause's true nodes, per edge type
    // [own][per_clause][SB]: bank 0 words, then bank 1 ...; 32-byte aligned (a word's 8 planes are moved as two vectors)
    uint32_t *ta = lds + ((size_t)(reach + (size_t)own_max * TE * NW - lds + 7) & ~(size_t)7);
    int32_t *wts = (int32_t *)(ta + (size_t)own_max * per_clause * SB);  // [own][K]
    int32_t *upd = wts + (size_t)own_max * K;                     // [own][K]
    int32_t *node_of = upd + (size_t)own_max * K;                 // [own]
    int32_t *incl_of = node_of + own_max;                         // [own]
    uint32_t *truth = (uint32_t *)(incl_of + own_max);            // [own][NW]
    int32_t *sums = (int32_t *)(truth + (size_t)own_max * NW);    // [K]
    int32_t *votes = sums + K;                                    // [K]
    uint32_t *seen = (uint32_t *)(votes + K);                     // [3][2][K] (see fit_persistent.h)
    uint32_t *hv_own = seen + 6 * K;                              // [own][MB] hypervector bits of the own clauses
    uint32_t *mlit = hv_own + (size_t)own_max * p.MB;             // [own][L][MC] message literal words of the picked node (not BIG)
    uint32_t *order = mlit;                                       // [literals] the literals, the ones that seldom hold first (BIG)
    // The workgroup's clauses: `own_max` slots, the first n_own of them taken - clauses g * own_max .. in order, or
    // what the table says (clauses dealt out by what they cost, k_fit_deep_deal below).  Everything that is
    // indexed by clause - automata, weights, hypervector bits, node types, random numbers - goes by own_id.
    int *own_id = (int *)(mlit + (BIG ? (size_t)p.literals : (size_t)own_max * L * MC));  // [own]
    uint32_t *queue_of_wave = (uint32_t *)(own_id + own_max);  // [waves][FIT_QUEUE] included literals waiting for their rows (BIG)
    __shared__ int n_own_shared;
    if (tid == 0) {
        int n = 0;
        for (int cl = 0; cl < own_max; ++cl) {
            const int c = p.perm ? p.perm[g * own_max + cl] : (g * own_max + cl < p.C ? g * own_max + cl : -1);
            if (c >= 0) own_id[n++] = c;
        }
        n_own_shared = n;
    }
    __syncthreads();
    const int n_own = n_own_shared;
    __shared__ int go_on;
    __shared__ int next_unit[2];  // waves take their units of work (a clause, or some words of one) from here: [0] layer 0, [1] a message layer

    // where the automata of own clause cl, word w of all its banks' words, live in global memory
    auto word_in_memory = [&](int cl, int w) -> uint32_t * {
        const int bank = w < LA ? 0 : 1 + (w - LA) / MC;
        const int wl = w < LA ? w : (w - LA) % MC, chunks = bank == 0 ? LA : MC;
        return p.bank[bank] + ((int64_t)own_id[cl] * chunks + wl) * B;
    };

    // own state -> LDS
    for (int k = tid; k < K; k += FITD_BLOCK) votes[k] = 0;
    for (int j = tid; j < 6 * K; j += FITD_BLOCK) seen[j] = 0u;
    for (int i = tid; i < n_own * per_clause * SB; i += FITD_BLOCK) {
        const int cl = i / (per_clause * SB), r = i - cl * per_clause * SB;
        const int w = r / SB, b = BIG ? B - 1 : r - w * SB;
        ta[i] = word_in_memory(cl, w)[b];
    }
    for (int i = tid; i < n_own * K; i += FITD_BLOCK) {
        const int cl = i / K, k = i - cl * K;
        wts[i] = p.weights[(int64_t)k * p.C + own_id[cl]];
    }
    for (int i = tid; i < n_own * p.MB; i += FITD_BLOCK) hv_own[i] = p.hv[(int64_t)own_id[i / p.MB] * p.MB + i % p.MB];
    if constexpr (BIG)
        for (int i = tid; i < p.literals; i += FITD_BLOCK) order[i] = p.order[i];
    if (tid == 0) go_on = 1, next_unit[0] = 0;
    lds_barrier();

    const int ones_row = p.literals + p.n_types;
    const size_t layer_words = (size_t)M * NW, slot_words = (size_t)L * layer_words;
    const size_t share_lo = (size_t)g * layer_words / G, share_hi = (size_t)(g + 1) * layer_words / G;
    // how the automaton words of the own clauses are spread over the waves: `parts` waves per clause
    const int parts0 = max(1, min(LA, WAVES / max(1, n_own))), chunk0 = (LA + parts0 - 1) / parts0;
#ifdef FITD_CLOCKS
    unsigned long long clk[16] = {}, last_ = wall_clock64();
#endif

    // the layer-0 rows of a graph (only the words that hold its nodes; not BIG), its edges and labels -> LDS
    // (threads t of nt take part)
    auto stage = [&](int ex_s, uint32_t *to, int t, int nt) {
        const int n_s = (int)p.n_nodes[ex_s];
        const int64_t base_s = (int64_t)p.node_index[ex_s];
        int32_t *y_s = (int32_t *)(to + p.rows_words + 2 * p.max_nodes + p.edge_cap);
        for (int k = t; k < K; k += nt) y_s[k] = p.encoded_Y[(int64_t)ex_s * K + k];
        if constexpr (!BIG) {
            const FitGraph fg_s = fit_graph_slot(p.tg, ex_s, n_s);
            const uint32_t *tile = p.tiles + (int64_t)fg_s.tile * p.tg.rows * p.tg.tw + fg_s.word0;
            const int words_s = fg_s.words, total = (p.literals + p.n_types + 1) * words_s;
            for (int at = t; at < total; at += nt) {
                const int r = at / words_s, w = at - r * words_s;
                to[at] = tile[(int64_t)r * p.tg.tw + w];
            }
        }
        if (p.has_edges && n_s > 0) {
            uint32_t *first_s = to + p.rows_words, *count_s = first_s + p.max_nodes, *pack_s = count_s + p.max_nodes;
            const uint32_t e0 = p.edge_index[base_s];
            const uint32_t total_edges = p.edge_index[base_s + n_s - 1] + p.n_edges[base_s + n_s - 1] - e0;
            for (int j = t; j < n_s; j += nt) {
                first_s[j] = p.edge_index[base_s + j] - e0;
                count_s[j] = p.n_edges[base_s + j];
            }
            const uint2 *pairs = (const uint2 *)p.edge + e0;
            for (uint32_t e = t; e < total_edges; e += nt) {
                const uint2 d = pairs[e];
                pack_s[e] = d.x | (d.y << 16);
            }
        }
    };
    // the next unit of work for this wave (clauses differ a lot in what they cost: a fixed share per wave leaves most waves idle)
    auto take_unit = [&](int which) {
        int u = 0;
        if (lane == 0) u = atomicAdd(&next_unit[which], 1);
        return __builtin_amdgcn_readfirstlane(u);
    };
    if (p.n_examples > 0) stage(p.first_example, lds, tid, FITD_BLOCK);
    lds_barrier();

    for (int i = 0; i < p.n_examples; ++i) {
        const int ex = p.first_example + i;
        const uint32_t step = p.first_step + (uint32_t)i;
        const int n = (int)p.n_nodes[ex];
        const int64_t base = (int64_t)p.node_index[ex];
        const FitGraph fg = fit_graph_slot(p.tg, ex, n);
        const int words = fg.words;
        const int slot = i % 3, slot_next = (i + 1) % 3;
        uint32_t *got_now = p.got + (size_t)slot * slot_words, *got_next = p.got + (size_t)slot_next * slot_words;
        unsigned long long *slot_sum = p.class_sum + (size_t)slot * K * FITP_SUM_PARTS * FITP_SUM_STRIDE;

        // ---- 0. the graph's edges (and layer-0 rows) are in LDS, fetched during the previous example
        uint32_t *rows0 = lds + (size_t)(i & 1) * staged_words;   // row r at rows0[r * words]
        const uint32_t *e_first = rows0 + p.rows_words, *e_count = e_first + p.max_nodes, *e_pack = e_count + p.max_nodes;
        const int32_t *y = (const int32_t *)(e_pack + p.edge_cap);
        const uint32_t *tile = p.tiles + (int64_t)fg.tile * p.tg.rows * p.tg.tw + fg.word0;  // (BIG: the rows in place)
        const int row_stride = BIG ? p.tg.tw : words;
        for (int at = tid; at < n_own * TE * NW; at += FITD_BLOCK) reach[at] = 0u;
        for (int cl = tid; cl < n_own; cl += FITD_BLOCK) incl_of[cl] = 0;
        // ---- 1. layer 0 (K1): truth of own clauses over the graph's nodes, lane = word; the include
        //         words of a clause are shared out over `parts0` waves, whose results meet in LDS.
        //         Truth starts as the clause's node-type row (K1 looks at nodes of the clause's type only).
        if constexpr (BIG) {
            // (clauses with many literals: the rows of a few literals that seldom hold, then the surviving
            // nodes against the whole include mask, as k_fit_eval does)
            const bool active = lane < words;
            for (int cl = take_unit(0); cl < n_own; cl = take_unit(0)) {
                int included;
                const uint32_t v = fit_clause_truth(ta + (size_t)cl * per_clause, 1, LA, p.filter, tile + (active ? lane : 0), row_stride,
                                                    p.literals, p.literals + own_id[cl] % p.n_types, ones_row, fg, n, FIT_WALK_ALL,
                                                    p.X + base * LA, order, active, lane, &included,
                                                    queue_of_wave + wave * FIT_QUEUE);
                if (lane < NW) truth[cl * NW + lane] = v;
                if (lane == 0) incl_of[cl] = included;
            }
            lds_barrier();
            FITD_TICK(0)
        } else {
            for (int at = tid; at < n_own * NW; at += FITD_BLOCK) {
                const int cl = at / NW, w = at - cl * NW;
                truth[at] = w < words ? rows0[(int64_t)(p.literals + own_id[cl] % p.n_types) * row_stride + w] : 0u;
            }
            lds_barrier();
            FITD_TICK(0)
            const bool active = lane < words;
            for (int u = wave; u < n_own * parts0; u += WAVES) {
                const int cl = u / parts0, part = u - cl * parts0;
                uint32_t acc = active ? truth[cl * NW + lane] : 0u;
                const uint32_t before = acc;
                fitd_and_rows<false>(ta + (size_t)cl * per_clause * SB + (SB - 1), SB, part * chunk0, min(LA, (part + 1) * chunk0), -1,
                              LA - 1, p.filter, (const uint32_t *)rows0 + (active ? lane : 0), row_stride, 0, 0, false, ones_row, acc,
                              &incl_of[cl], lane);
                if (active && acc != before) atomicAnd(&truth[cl * NW + lane], acc);
            }
            lds_barrier();
            if (fg.shift != 0 || fg.mask != 0xFFFFFFFFu) {  // several graphs share a word: keep this graph's bits
                for (int cl = tid; cl < n_own; cl += FITD_BLOCK) truth[cl * NW] = (truth[cl * NW] >> fg.shift) & fg.mask;
                lds_barrier();
            }
        }
        FITD_TICK(1)

        // ---- 2. the message layers
        bool alive = true;
        for (int l = 0; l < L && alive; ++l) {
            uint32_t *got_l = got_now + (size_t)l * layer_words;
            unsigned long long *arrived = p.arrived + (size_t)l * FITD_PARTS * FITD_STRIDE;
            const unsigned long long everyone = (unsigned long long)(i + 1) * (unsigned long long)G;
            // a. what the own clauses make the nodes receive
            if (p.has_edges && n > 0) {
                if (p.by_masks && n_own > 2) {
                    // 32 clauses at a time: per node the clauses that are true there as a mask, the masks carried
                    // along the edges (one pass over the edges whatever the number of clauses), and the masks that
                    // arrived turned back into a row of nodes per clause and edge type.  (The masks use the
                    // LDS of the received rows, which are not there yet.)
                    uint32_t *mask_at = mrows, *mask_in = mrows + p.max_nodes;  // [max_nodes], [TE][max_nodes]
                    for (int first_cl = 0; first_cl < n_own; first_cl += 32) {
                        const int nb = min(32, n_own - first_cl);
                        for (int u = tid >> 5; u < words; u += FITD_BLOCK / 32) {  // half a wave per word of nodes
                            const int b = lane & 31;
                            const uint32_t t = fitd_transpose32(b < nb ? truth[(first_cl + b) * NW + u] : 0u, lane);
                            if (u * 32 + b < n) mask_at[u * 32 + b] = t;
                        }
                        for (int at = tid; at < TE * p.max_nodes; at += FITD_BLOCK) mask_in[at] = 0u;
                        lds_barrier();
                        for (int src = tid; src < n; src += FITD_BLOCK) {
                            const uint32_t mask = mask_at[src];
                            if (mask == 0u) continue;
                            const uint32_t first = e_first[src], count = e_count[src];
                            for (uint32_t e = 0; e < count; ++e) {
                                const uint32_t d = e_pack[first + e], dst = d & 0xFFFFu, type = d >> 16;
                                atomicOr(&mask_in[type * p.max_nodes + dst], mask);
                            }
                        }
                        lds_barrier();
                        for (int u = tid >> 5; u < TE * words; u += FITD_BLOCK / 32) {  // half a wave per type and word of nodes
                            const int type = u / words, w = u - type * words, k = lane & 31;
                            const uint32_t t = fitd_transpose32(w * 32 + k < n ? mask_in[type * p.max_nodes + w * 32 + k] : 0u, lane);
                            if (k < nb) reach[((first_cl + k) * TE + type) * NW + w] = t;
                        }
                        lds_barrier();
                    }
                } else {
                    for (int at = tid; at < n_own * n; at += FITD_BLOCK) {
                        const int cl = at / n, src = at - cl * n;
                        if (!((truth[cl * NW + (src >> 5)] >> (src & 31)) & 1u)) continue;
                        const uint32_t first = e_first[src], count = e_count[src];
                        for (uint32_t e = 0; e < count; ++e) {
                            const uint32_t d = e_pack[first + e], dst = d & 0xFFFFu, type = d >> 16;
                            atomicOr(&reach[(cl * TE + (int)type) * NW + (dst >> 5)], 1u << (dst & 31));
                        }
                    }
                    lds_barrier();
                }
                FITD_TICK(6)
                for (int at = tid; at < n_own * TE * words; at += FITD_BLOCK) {
                    const int cl = at / (TE * words), r = at - cl * TE * words;
                    const int type = r / words, w = r - type * words;
                    const uint32_t v = reach[(cl * TE + type) * NW + w];
                    if (v != 0u)
                        for (int j = 0; j < p.MB; ++j) {
                            const uint32_t row = (hv_own[cl * p.MB + j] + (uint32_t)type) % (uint32_t)M;
                            __hip_atomic_fetch_or(&got_l[(size_t)row * NW + w], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                }
            }
            FITD_TICK(7)
            __builtin_amdgcn_s_waitcnt(FITP_WAIT_VMEM);  // the ORs have been carried out where every workgroup sees them
            asm volatile("" ::: "memory");
            lds_barrier();
            FITD_TICK(2)
            if (tid == 0)
                __hip_atomic_fetch_add(&arrived[(g % FITD_PARTS) * FITD_STRIDE], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (wave == 0) {
                const bool ok = fitd_wait(arrived, everyone, p.abort_flag, p.spin_limit, p.wait_ticks, p.force_abort, lane);
                if (lane == 0) go_on = ok ? 1 : 0;
            } else {
                // (meanwhile) this group's share of the slot the next example will send into; the next
                // example's rows and edges
                for (size_t at = share_lo + (size_t)(tid - 64); at < share_hi; at += FITD_BLOCK - 64)
                    __hip_atomic_store(&got_next[(size_t)l * layer_words + at], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                for (int at = tid - 64; at < n_own * TE * NW; at += FITD_BLOCK - 64) reach[at] = 0u;
                if (l == 0 && i + 1 < p.n_examples) stage(ex + 1, lds + (size_t)((i + 1) & 1) * staged_words, tid - 64, FITD_BLOCK - 64);
            }
            lds_barrier();
            FITD_TICK(3)
            if (!go_on) {
                alive = false;
                break;
            }
            // b. the received rows -> LDS, a window at a time, and K2 for own clauses on the window's literals
            for (int r0 = 0; r0 < M; r0 += WR) {
                const int r1 = min(M, r0 + WR), w_first = r0 >> 5, window_words = (r1 - r0) >> 5;
                {
                    const unsigned long long *from = (const unsigned long long *)(got_l + (size_t)r0 * NW);  // (32 NW is even, the rows 8-byte aligned)
                    unsigned long long *to = (unsigned long long *)mrows;
                    const int pairs = (r1 - r0) * NW / 2;
                    for (int at0 = tid; at0 < pairs; at0 += 8 * FITD_BLOCK) {
                        unsigned long long v[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u)
                            v[u] = at0 + u * FITD_BLOCK < pairs
                                       ? __hip_atomic_load(&from[at0 + u * FITD_BLOCK], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                       : 0ull;
#pragma unroll
                        for (int u = 0; u < 8; ++u)
                            if (at0 + u * FITD_BLOCK < pairs) to[at0 + u * FITD_BLOCK] = v[u];
                    }
                    if (tid == 0) next_unit[1] = 0;
                }
                lds_barrier();
                FITD_TICK(4)
                {
                    const bool active = lane < NW;
                    const uint32_t *col = mrows + (active ? lane : 0);
                    const int parts1 = max(1, min(window_words, WAVES / max(1, n_own)));
                    const int chunk1 = (window_words + parts1 - 1) / parts1;
                    const int units = n_own * parts1;
                    const bool queued = units > WAVES;  // (a unit per wave at most: nothing to balance)
                    for (int u = queued ? take_unit(1) : wave; u < units; u = queued ? take_unit(1) : units) {
                        const int cl = u / parts1, part = u - cl * parts1;
                        uint32_t acc = active ? truth[cl * NW + lane] : 0u;
                        const uint32_t before = acc;
                        const uint32_t *inc = ta + ((size_t)cl * per_clause + LA + (size_t)l * MC) * SB + (SB - 1);
                        const int lo = w_first + part * chunk1, hi = min(w_first + window_words, lo + chunk1);
                        // (2 M is a multiple of 32: the last word has no tail to mask) the words of the positive literals and,
                        // in the same pass, those of the negated ones (MW words further on)
                        fitd_and_rows<BIG>(inc, SB, lo, hi, MW, -1, 0u, col, NW, r0, M, true, r0, acc, &incl_of[cl], lane);
                        if (active && acc != before) atomicAnd(&truth[cl * NW + lane], acc);
                    }
                }
                if constexpr (BIG) {
                    // what the nodes of this group's share received, node-major: bit b of word j of node v = bit v of row 32 j + b
                    const int v_lo = (int)((int64_t)g * n / G), v_hi = (int)((int64_t)(g + 1) * n / G);
                    uint32_t *vec_l = p.vec + (size_t)l * p.max_nodes * MW;
                    for (int at = tid; at < (v_hi - v_lo) * window_words; at += FITD_BLOCK) {
                        const int v = v_lo + at / window_words, j = at % window_words;
                        uint32_t word = 0u;
                        for (int b = 0; b < 32; ++b) word |= ((mrows[(j * 32 + b) * NW + (v >> 5)] >> (v & 31)) & 1u) << b;
                        __hip_atomic_store(&vec_l[(size_t)v * MW + w_first + j], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
                lds_barrier();
                FITD_TICK(5)
            }
        }
        if (!alive) break;

        // ---- 3. node pick (K7) and votes (K6)
        for (int cl = wave; cl < n_own; cl += WAVES) {
            const int c = own_id[cl];
            const uint32_t v = lane < NW ? truth[cl * NW + lane] : 0u;
            const int pc = __popc(v);
            int true_nodes, before;
            wave_count_scan(pc, lane, &true_nodes, &before);
            bool fired = true_nodes > 0;
            int node = -1;
            if (n == 0) {
                fired = true;  // the reference's arithmetic for a graph without nodes (kernels.py:289-295)
            } else if (fired) {
                philox_out r = philox4x32_10((uint32_t)c, 0u, step, GTM_TAG_CLAUSE_NODE, p.k0, p.k1);
                const int pick = (int)(((uint64_t)r.v[0] * (uint64_t)true_nodes) >> 32);
                const bool mine_is = pick >= before && pick < before + pc;
                int candidate = 0;
                if (mine_is) {
                    uint32_t t = v;
                    for (int j = before; j < pick; ++j) t &= t - 1;
                    candidate = lane * 32 + __ffs(t) - 1;
                }
                const unsigned long long owner = __ballot(mine_is);
                node = __builtin_amdgcn_readlane(candidate, __ffsll((long long)owner) - 1);
            }
            if (lane == 0) node_of[cl] = node;
            if (fired)
                for (int k = lane; k < K; k += 64) atomicAdd(&votes[k], wts[cl * K + k]);  // LDS
        }
        // the next slot's share is cleared (and the node-major words are out) before this group arrives
        __builtin_amdgcn_s_waitcnt(FITP_WAIT_VMEM);
        asm volatile("" ::: "memory");
        lds_barrier();
        FITD_TICK(9)

        // ---- 4. class sums across the device (the protocol of fit_persistent.h)
        for (int k = tid; k < K; k += FITD_BLOCK) {
            __hip_atomic_fetch_add(&slot_sum[(k * FITP_SUM_PARTS + (g % FITP_SUM_PARTS)) * FITP_SUM_STRIDE],
                                   FITP_ARRIVED + (unsigned long long)(long long)votes[k], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            votes[k] = 0;
        }
        uint32_t x_first = 0u;  // the literal word of this thread's first automaton word of bank 0 (see step 6)
        if constexpr (!BIG) {
            // the message literals of the picked nodes: bit `node` of the layer's received rows, packed as
            // kernels.py:592-615 packs them (the negated half is the complement); done, like the fetch of the
            // picked nodes' literal words, while the sums travel
            for (int at = FITD_BLOCK - 1 - tid; at < n_own * L * MW; at += FITD_BLOCK) {
                const int cl = at / (L * MW), r = at - cl * L * MW;
                const int l = r / MW, j = r - l * MW;
                const int node = node_of[cl];
                uint32_t word = 0u;
                if (node >= 0) {
                    if (l == L - 1) {
                        for (int b = 0; b < 32; ++b) word |= ((mrows[(j * 32 + b) * NW + (node >> 5)] >> (node & 31)) & 1u) << b;
                    } else {
                        const uint32_t *rows_l = got_now + (size_t)l * layer_words;
                        for (int b = 0; b < 32; ++b)
                            word |= ((fitd_load(&rows_l[(size_t)(j * 32 + b) * NW + (node >> 5)]) >> (node & 31)) & 1u) << b;
                    }
                }
                mlit[((size_t)cl * L + l) * MC + j] = word;
                mlit[((size_t)cl * L + l) * MC + MW + j] = ~word;
            }
            if (tid < n_own * per_clause) {
                const int cl = tid / per_clause, w = tid - cl * per_clause;
                if (w < LA && node_of[cl] >= 0) x_first = p.X[(base + node_of[cl]) * LA + w];
            }
        }
        if (tid < K) {
            const int k = tid;
            const unsigned long long everyone = (unsigned long long)G;
            uint32_t *seen_slot = seen + (size_t)slot * 2 * K;
            const unsigned long long seen_own = ((unsigned long long)seen_slot[K + k] << 32) | seen_slot[k];
            uint32_t polls = 0;
            unsigned long long waiting_since = 0ull;
            unsigned long long word = 0ull;
            bool ok = !p.force_abort;
            if (!ok) __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            while (ok) {
                unsigned long long all = 0ull;
#pragma unroll
                for (int s = 0; s < FITP_SUM_PARTS; ++s)
                    all += __hip_atomic_load(&slot_sum[(k * FITP_SUM_PARTS + s) * FITP_SUM_STRIDE], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
                word = all;
                if ((((word - seen_own + FITP_HALF) >> 48) & 0xFFFFull) == everyone) break;
                if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 ||
                    fit_wait_is_over(polls, p.spin_limit, waiting_since, p.wait_ticks)) {
                    __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ok = false;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            if (!ok) go_on = 0;
            sums[k] = (int32_t)(long long)(word - seen_own - (everyone << 48));
            seen_slot[k] = (uint32_t)word, seen_slot[K + k] = (uint32_t)(word >> 32);
        }
        lds_barrier();
        FITD_TICK(10)
        if (!go_on) break;

        // ---- 5. feedback decisions (K8) and weights
        for (int j = tid; j < n_own * K; j += FITD_BLOCK) {
            const int cl = j / K, k = j - cl * K;
            int cs = sums[k];
            cs = cs > p.T ? p.T : (cs < -p.T ? -p.T : cs);
            const int yk = y[k];
            const int target = 1 - 2 * (cs > yk);
            int w = wts[j];
            const int sign = (w >= 0) - (w < 0);
            int err = yk - cs;
            err = err < 0 ? -err : err;
            philox_out r = philox4x32_10((uint32_t)own_id[cl], (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, p.k0, p.k1);
            const bool skip = (target == -1 && (uint64_t)r.v[0] >= p.q_thr) ||
                              ((uint64_t)r.v[1] * (uint64_t)(2 * (int64_t)p.T) >= ((uint64_t)err << 32));
            const int u = skip ? 0 : target * sign;
            const bool fired = node_of[cl] != -1;
            if (u > 0 && fired && (w < 0 ? -(int64_t)w : (int64_t)w) < 2147483647) {
                wts[j] = w + sign;
            } else if (u < 0 && fired) {
                w -= sign;
                if (p.negative == 0 && w < 1) w = 1;
                wts[j] = w;
            }
            upd[j] = u;
        }
        lds_barrier();
        FITD_TICK(11)

        // ---- 6. Type I / II feedback on every bank (K9, K10), one thread per automaton word
        if constexpr (!BIG) {
            for (int at = tid; at < n_own * per_clause; at += FITD_BLOCK) {
                const int cl = at / per_clause, w = at - cl * per_clause;
                const int32_t *u_of = upd + cl * K;
                bool any = false;
                for (int k = 0; k < K; ++k) any |= u_of[k] != 0;
                if (!any) continue;
                const int node = node_of[cl];
                const bool fired = node != -1;
                const bool within = incl_of[cl] <= p.max_included;
                const int bank = w < LA ? 0 : 1 + (w - LA) / MC;
                const int wl = w < LA ? w : (w - LA) % MC;
                uint32_t x = 0u;
                if (fired) x = bank != 0 ? mlit[((size_t)cl * L + (bank - 1)) * MC + wl] : at == tid ? x_first : p.X[(base + node) * LA + wl];
                feedback_word<MAXB>(ta + (size_t)at * B, B, K, u_of, 1, fired, within, p.boost, x, p.k0, p.k1, (uint32_t)own_id[cl],
                                    (uint32_t)wl, step, (uint32_t)bank, p.thr16[bank]);
            }
        } else {
            // eight words at a time: their literal words are fetched first (from X, or node-major from `vec`), so that
            // the fetches travel together
            for (int at0 = tid; at0 < n_own * per_clause; at0 += 8 * FITD_BLOCK) {
                uint32_t x[8];
                bool busy[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int at = at0 + u * FITD_BLOCK;
                    x[u] = 0u, busy[u] = false;
                    if (at >= n_own * per_clause) continue;
                    const int cl = at / per_clause, w = at - cl * per_clause;
                    const int32_t *u_of = upd + cl * K;
                    for (int k = 0; k < K; ++k) busy[u] |= u_of[k] != 0;
                    const int node = node_of[cl];
                    if (!busy[u] || node < 0) continue;
                    if (w < LA) {
                        x[u] = p.X[(base + node) * LA + w];
                    } else {
                        const int bank = 1 + (w - LA) / MC, wl = (w - LA) % MC;
                        const uint32_t word = fitd_load(&p.vec[((size_t)(bank - 1) * p.max_nodes + node) * MW + (wl < MW ? wl : wl - MW)]);
                        x[u] = wl < MW ? word : ~word;
                    }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (!busy[u]) continue;
                    const int at = at0 + u * FITD_BLOCK;
                    const int cl = at / per_clause, w = at - cl * per_clause;
                    const int bank = w < LA ? 0 : 1 + (w - LA) / MC;
                    const int wl = w < LA ? w : (w - LA) % MC;
                    // (the include plane's copy in LDS follows)
                    ta[at] = feedback_word<MAXB>(word_in_memory(cl, w), B, K, upd + cl * K, 1, node_of[cl] != -1,
                                                 incl_of[cl] <= p.max_included, p.boost, x[u], p.k0, p.k1, (uint32_t)own_id[cl],
                                                 (uint32_t)wl, step, (uint32_t)bank, p.thr16[bank]);
                }
            }
        }
        if (tid == 0) next_unit[0] = 0;
        lds_barrier();
        FITD_TICK(12)
    }
#ifdef FITD_CLOCKS
    if (g == 0 && tid == 0 && p.clocks)
        for (int k = 0; k < 16; ++k) p.clocks[k] = clk[k];
#endif
    lds_barrier();
    // own state -> global memory (also after an abort: the host puts the model back as it was)
    if constexpr (!BIG)
        for (int i = tid; i < n_own * per_clause * B; i += FITD_BLOCK) {
            const int cl = i / (per_clause * B), r = i - cl * per_clause * B;
            const int w = r / B, b = r - w * B;
            word_in_memory(cl, w)[b] = ta[i];
        }
    for (int i = tid; i < n_own * K; i += FITD_BLOCK) {
        const int cl = i / K, k = i - cl * K;
        p.weights[(int64_t)k * p.C + own_id[cl]] = wts[i];
    }
}
