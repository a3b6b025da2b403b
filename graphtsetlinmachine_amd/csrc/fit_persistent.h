// A whole run of training examples (the loop at tm.py:669-747) of a depth-1
// model in ONE cooperative launch.
//
// Each workgroup owns a contiguous range of clauses for the whole run and keeps
// their automata (all bit planes) and weights in LDS; they go back to global
// memory once, at the end.  Per example a workgroup
//   1. evaluates its clauses on the graph's literal-major rows (staged in LDS;
//      the next graph's rows, literal words and labels are loaded straight into
//      the other LDS buffers while waiting at the barrier), picks the nodes, and
//      adds its clauses' votes to the class sums in global memory;
//   2. meets the other workgroups at a device-wide barrier (the class sums are
//      the only thing that crosses clause boundaries, kernels.py:310-315);
//   3. decides the feedback and updates its automata and weights in LDS.
// Class sums and barrier are one thing: class k has a 64-bit word (kept as
// FITP_SUM_PARTS partial words that a reader adds up, since the memory system
// carries out the adds to one word one after the other) to which every
// workgroup adds (1 << 48) + its share with one device-scope atomic, and which it
// then polls.  Nothing else is ever done to the word - no reset, no store - so
// per-location coherence is all the protocol needs: nothing has to be ordered
// against a separate barrier word and no cache is flushed or invalidated.  What an
// example contributed is the word now minus the word as it stood when its last use
// was complete (each polling thread remembers that value): modulo 2^64 that
// difference is arrivals * 2^48 + sum, whatever borrows negative shares caused, so
// with |sum| < 2^47 the arrivals are (difference + 2^47) >> 48 and, once they equal
// the number of workgroups, the sum is the rest.  The words live in a ring of three
// slots, each partial word in a cache line of its own (the adds and polls go to
// different memory channels): a workgroup can be one example ahead of the
// slowest one, never three.  Thread k of a workgroup polls the word of class k.
// The workgroup's barriers order LDS traffic only, so none of them waits for the
// adds or for the loads of the next graph.
//
// The wait is bounded (a few seconds of the device's wall clock; a number of polls
// in tests): a workgroup whose wait runs out raises the abort flag and every
// workgroup leaves the loop at its next check, so the grid always drains.  The
// host then puts the model back as it was and trains the examples by launches per
// example instead.
#pragma once

constexpr int FITP_BLOCK = 1024;  // 16 waves: one clause per wave in flight, four waves per SIMD hide each other's latencies

// A device-wide wait gives up after `spin_limit` polls or `wait_ticks` ticks of the wall clock (constant
// rate, whatever the shader clock does), whichever comes first.  The clock is a memory instruction of its
// own, so it is only looked at every 256th poll: an ordinary wait (a few polls) never reads it.
__device__ __forceinline__ bool fit_wait_is_over(uint32_t &polls, uint32_t spin_limit, unsigned long long &since,
                                                 unsigned long long wait_ticks) {
    if (++polls > spin_limit) return true;
    if ((polls & 255u) == 0u) {
        const unsigned long long now = wall_clock64();
        if (since == 0ull)
            since = now;
        else if (now - since > wait_ticks)
            return true;
    }
    return false;
}

struct FitPersistParams {
    // data set
    const uint32_t *tiles;
    const uint32_t *X;
    const uint32_t *node_index;
    const uint32_t *n_nodes;
    const int32_t *encoded_Y;
    TileGeom tg;
    int first_example, n_examples;
    uint32_t first_step;
    // model
    uint32_t *bank;
    int32_t *weights;
    int literals, n_types, C, LA, B, K, T, negative, boost, max_included;
    uint32_t filter, thr16, k0, k1;
    uint64_t q_thr;
    // coordination
    unsigned long long *class_sum;  // [3][K][FITP_SUM_PARTS] words FITP_SUM_STRIDE apart, zero on entry (K <= FITP_BLOCK)
    uint32_t *abort_flag;           // [1], zero on entry
    uint32_t spin_limit;  // polls after which a wait gives up (tests; 2^32 - 1 otherwise: the clock bounds the wait)
    unsigned long long wait_ticks;  // ticks of the device's wall clock after which a wait gives up
    int force_abort;      // give up at the first wait without looking (exercises the drain path)
    int clauses_per_group;
    int rows_words;       // LDS words of one staged graph: (literals + n_types + 1) * max slot words
    int max_words;        // words per graph slot that can hold nodes
    const uint32_t *order;  // literals sorted by how often they hold in the data set, rarest first
    int x_words;          // LDS words of one graph's node-major literal words: max nodes * LA
    const uint32_t *node_type;  // [total nodes]
    int direct;           // graphs of at most FITP_DIRECT_NODES nodes: every node is tested on its own literal words, no rows are staged
};

__device__ __forceinline__ void fitp_stage_rows(const FitPersistParams &p, const FitGraph &fg, uint32_t *dst, int tid) {
    const uint32_t *tile = p.tiles + (int64_t)fg.tile * p.tg.rows * p.tg.tw + fg.word0;
    const int words = fg.words;
    const int total = (p.literals + p.n_types + 1) * words;
    // element i = r * words + w; a thread visits i = tid, tid + FITP_BLOCK, ...: (r, w) advance without dividing
    const int dr = FITP_BLOCK / words, dw = FITP_BLOCK - dr * words;
    int r = tid / words, w = tid - r * words;
    for (int base = tid; base < total; base += FITP_BLOCK * 8) {
        uint32_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            v[u] = base + u * FITP_BLOCK < total ? tile[(int64_t)r * p.tg.tw + w] : 0u;
            r += dr;
            w += dw;
            if (w >= words) {
                w -= words;
                ++r;
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (base + u * FITP_BLOCK < total) dst[base + u * FITP_BLOCK] = v[u];
    }
}

constexpr unsigned long long FITP_HALF = 1ull << 47;      // class sums are smaller than this in magnitude
constexpr unsigned long long FITP_ARRIVED = 1ull << 48;   // one arrival in bits 48..63
constexpr int FITP_SUM_STRIDE = 16;                      // 64-bit words between two class-sum words (one per 128-byte line)
// A class sum is kept as this many partial words; group g adds to part g % FITP_SUM_PARTS and the
// reader adds the parts up (the protocol is linear in the word). Adds to one word are carried out
// one after the other by the memory system, so fewer groups per word shorten the exchange.
constexpr int FITP_SUM_PARTS = 16;
constexpr int FITP_WALK_ALL = 24;   // clauses with at most this many literals AND all their rows
constexpr int FITP_FILTER_ROWS = 16;  // rows the others AND before testing the surviving nodes
constexpr int FITP_DIRECT_NODES = 2;  // data sets whose graphs have at most this many nodes skip the literal rows altogether
constexpr int FITP_FEW_NODES = 2;     // up to this many surviving nodes are tested one by one, more are filtered further

// One 32-bit word per lane from global memory straight into LDS (no register holds it meanwhile):
// lane l's word lands at dst_of_wave[l]; dst_of_wave must be the same for the whole wave. The words
// are there once the wave has waited for its vector-memory counter (FITP_WAIT_VMEM) and, for other
// waves, after the barrier that follows.
__device__ __forceinline__ void fitp_load_to_lds(const uint32_t *src, uint32_t *dst_of_wave) {
    __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) uint32_t *)dst_of_wave, 4, 0, 0);
}
// Between LDS writes of some lanes of a wave and reads of them by other lanes of the same wave (the
// hardware carries out a wave's LDS accesses in order; this keeps the compiler from reordering them).
__device__ __forceinline__ void fitp_wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}
constexpr int FITP_WAIT_VMEM = 0x0F70;  // s_waitcnt vmcnt(0) (export and LDS counters left alone)

// MAXB: bit planes of an automaton the kernel keeps in registers while updating a word (>= B).
template <int MAXB>
__global__ __launch_bounds__(FITP_BLOCK) void k_fit_persistent(FitPersistParams p) {
    extern __shared__ uint32_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int WAVES = FITP_BLOCK / 64;
    const int c0 = blockIdx.x * p.clauses_per_group;
    const int n_own = min(p.clauses_per_group, p.C - c0);
    const int LA = p.LA, B = p.B, K = p.K;
    const int own_max = p.clauses_per_group;

    // LDS carve-up
    uint32_t *rows_buf[2] = {lds, lds + p.rows_words};
    uint32_t *ta = lds + 2 * p.rows_words;                     // [own][LA][B]
    int32_t *wts = (int32_t *)(ta + (size_t)own_max * LA * B);  // [own][K]
    int32_t *upd = wts + (size_t)own_max * K;                  // [own][K]
    int32_t *node_of = upd + (size_t)own_max * K;              // [own]
    int32_t *incl_of = node_of + own_max;                      // [own]
    int32_t *sums = incl_of + own_max;                         // [K] class sums of the example
    int32_t *votes = sums + K;                                 // [K] this group's share of the class sums
    uint32_t *gate = (uint32_t *)(votes + K);                  // [own][K][2] random words of the feedback gates
    uint32_t *fbits = gate + 2 * (size_t)own_max * K;          // [own][LA][K] Type I feedback bits
    int32_t *pair_list = (int32_t *)(fbits + (size_t)own_max * LA * K);  // [own * K] (clause, class) pairs with Type I feedback
    uint32_t *x_buf[2] = {(uint32_t *)(pair_list + (size_t)own_max * K),
                          (uint32_t *)(pair_list + (size_t)own_max * K) + p.x_words};  // [nodes][LA] of the graph
    uint32_t *order_lds = x_buf[1] + p.x_words;                 // [literals]
    // thread k < K: its class-sum word as it stood when each of the three
    // slots was last complete (all zero before the first use): [slot][low, high][K]
    uint32_t *seen = order_lds + p.literals;
    uint32_t *y_buf[2] = {seen + 6 * K, seen + 7 * K};        // [K] labels of this and the next example
    __shared__ int go_on, n_pairs;
    __shared__ uint32_t after_lds[2];
    __shared__ uint32_t types_lds[2][FITP_DIRECT_NODES];  // node types of this and the next graph (direct evaluation)

    // own state -> LDS
    for (int k = tid; k < K; k += FITP_BLOCK) votes[k] = 0;
    for (int i = tid; i < n_own * LA * B; i += FITP_BLOCK) ta[i] = p.bank[(int64_t)c0 * LA * B + i];
    for (int i = tid; i < n_own * K; i += FITP_BLOCK) {
        int cl = i / K, k = i - cl * K;
        wts[i] = p.weights[(int64_t)k * p.C + c0 + cl];
    }
    const int last = p.first_example + p.n_examples - 1;
    int n_now = 0, n_next = 0;          // node counts of example i and i + 1
    uint32_t base_now = 0, base_next = 0;  // node_index of example i and i + 1
    if (p.n_examples > 0) {
        n_now = (int)p.n_nodes[p.first_example];
        base_now = p.node_index[p.first_example];
        const int e1 = min(p.first_example + 1, last);
        n_next = (int)p.n_nodes[e1];
        base_next = p.node_index[e1];
        FitGraph fg0 = fit_graph_slot(p.tg, p.first_example, n_now);
        if (!p.direct) fitp_stage_rows(p, fg0, rows_buf[0], tid);
        for (int at = tid; at < n_now * LA; at += FITP_BLOCK) x_buf[0][at] = p.X[(int64_t)base_now * LA + at];
        if (p.direct && tid < n_now) types_lds[0][tid] = p.node_type[base_now + tid];
        for (int k = tid; k < K; k += FITP_BLOCK) y_buf[0][k] = (uint32_t)p.encoded_Y[(int64_t)p.first_example * K + k];
    }
    for (int l = tid; l < p.literals; l += FITP_BLOCK) order_lds[l] = p.order[l];
    for (int j = tid; j < 6 * K; j += FITP_BLOCK) seen[j] = 0u;
    lds_barrier();

    const int ones_row = p.literals + p.n_types;
    // one small clause per wave: the feedback of a step runs inside the clause's wave
    const bool wave_local = own_max <= WAVES && K * LA <= 256;
    int div_words = 0, div_dr = 0, div_r0 = 0;
    // The threads that add the group's votes to the device-wide class sums and then poll for them are the first K
    // of the LAST wave when K <= 64; that wave requests none of the next graph's words and draws no random
    // numbers, so its polling starts at once and runs beside the other waves' work instead of after its own share.
    const bool poll_apart = K <= 64;
    const int poll0 = poll_apart ? (WAVES - 1) * 64 : 0;         // the first polling thread
    const int loaders = poll_apart ? poll0 : FITP_BLOCK;        // threads 0 .. loaders - 1 request the next graph's words
    for (int i = 0; i < p.n_examples; ++i) {
        const int ex = p.first_example + i;
        const uint32_t step = p.first_step + (uint32_t)i;
        const FitGraph fg = fit_graph_slot(p.tg, ex, n_now);
        const uint32_t *rows = rows_buf[i & 1];
        unsigned long long *slot_now = p.class_sum + (size_t)(i % 3) * K * FITP_SUM_PARTS * FITP_SUM_STRIDE;

        // ---- 0. the next graph's slot; the sizes of the graph after it are requested
        const bool has_next = i + 1 < p.n_examples;
        const FitGraph fn = fit_graph_slot(p.tg, has_next ? ex + 1 : ex, has_next ? n_next : n_now);
        const int next_total = has_next && !p.direct ? (p.literals + p.n_types + 1) * fn.words : 0;
        const uint32_t *x_now = x_buf[i & 1];
        // node count and first node of the graph after the next, fetched by two threads with vector
        // loads (scalar loads share their counter with LDS: the evaluation's first LDS read would wait
        // for them) and handed over through LDS at the end of the step
        const int e2 = min(ex + 2, last);
        uint32_t after = 0u;
        if (tid < 2) after = (tid == 0 ? p.n_nodes : p.node_index)[e2];
        uint32_t type_ahead = 0u;
        if (p.direct && has_next && tid < n_next) type_ahead = p.node_type[base_next + tid];

        // ---- 1. evaluate own clauses (K1 + K7), votes (K6)
        const bool active = lane < fg.words;
        const uint32_t *col = rows + (active ? lane : 0);
        const int stride = fg.words;
        for (int cl = wave; cl < n_own; cl += WAVES) {
            const int c = c0 + cl;
            const uint32_t *inc = ta + (size_t)cl * LA * B + (B - 1);
            uint32_t acc = active && !p.direct ? col[(p.literals + c % p.n_types) * stride] : 0u;
            int included = 0;
            uint32_t first_words = 0;
            for (int w0 = 0; w0 < LA; w0 += 64) {
                uint32_t mine = w0 + lane < LA ? inc[(w0 + lane) * B] : 0u;
                if (w0 + lane == LA - 1) mine &= p.filter;
                if (w0 == 0) first_words = mine;
                included += wave_sum_small(__popc(mine));
            }
            // A clause with many literals ANDs only the rows of its FITP_FILTER_ROWS rarest ones and then
            // tests the few nodes that are left against its whole include mask on the nodes' own words.
            const bool filter_only = included > FITP_WALK_ALL && n_now > 0 && !p.direct;
            bool all_rows = false;  // every included literal's row has been applied: acc is the clause's truth
            if (filter_only) {
                int budget = FITP_FILTER_ROWS;
                bool stop = false;
                // The included literals in rarest-first order, 256 ranks at a time: the four LDS reads
                // of the ranks and the four of the include words are each issued together (a clause
                // whose rare literals are few would otherwise pay two LDS round trips per 64 ranks).
                for (int g0 = 0; g0 < p.literals && !stop; g0 += 256) {
                    uint32_t lit4[4];
                    unsigned long long m4[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int r = g0 + 64 * u + lane;
                        lit4[u] = r < p.literals ? order_lds[r] : 0u;
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int r = g0 + 64 * u + lane;
                        uint32_t word = inc[(lit4[u] >> 5) * B];
                        if ((int)(lit4[u] >> 5) == LA - 1) word &= p.filter;
                        m4[u] = __ballot(r < p.literals && ((word >> (lit4[u] & 31u)) & 1u));
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        unsigned long long picked = m4[u];  // lanes whose literal is included and not applied yet
                        const uint32_t lit = lit4[u];
                        while (picked != 0ull && !stop) {
                            if (budget <= 0) {
                                // a few surviving nodes are cheapest tested one by one; more than that, and 8 more
                                // rows (one LDS round trip) remove most of them at the price of testing one
                                // (counted as lanes with a survivor, twice those with several: an estimate is enough)
                                if (n_now <= FITP_FEW_NODES) {
                                    stop = true;
                                    break;
                                }
                                const int mine = active ? __popc((acc >> fg.shift) & fg.mask) : 0;
                                const int left = __popcll(__ballot(mine > 0)) + __popcll(__ballot(mine > 1));
                                if (left <= FITP_FEW_NODES) {
                                    stop = true;
                                    break;
                                }
                                budget = 8;
                            }
                            int row[8];
#pragma unroll
                            for (int v8 = 0; v8 < 8; ++v8) {
                                row[v8] = picked ? (int)__builtin_amdgcn_readlane(lit, __ffsll((long long)picked) - 1) : ones_row;
                                picked &= picked - 1;
                            }
                            uint32_t r8[8];
#pragma unroll
                            for (int v8 = 0; v8 < 8; ++v8) r8[v8] = col[row[v8] * stride];
#pragma unroll
                            for (int v8 = 0; v8 < 8; ++v8) acc &= r8[v8];
                            budget -= 8;
                        }
                    }
                }
                all_rows = !stop;  // every included literal's row has been applied
            } else if (!p.direct) {
                for (int w0 = 0; w0 < LA; w0 += 64) {
                    uint32_t mine = w0 == 0 ? first_words : (w0 + lane < LA ? inc[(w0 + lane) * B] : 0u);
                    if (w0 != 0 && w0 + lane == LA - 1) mine &= p.filter;
                    unsigned long long nonzero = __ballot(mine != 0);
                    while (nonzero) {
                        const int wl = __ffsll((long long)nonzero) - 1;
                        nonzero &= nonzero - 1;
                        uint32_t m = __builtin_amdgcn_readlane(mine, wl);
                        const int base = (w0 + wl) << 5;
                        while (m) {
                            int row[8];
#pragma unroll
                            for (int u = 0; u < 8; ++u) {
                                row[u] = m ? base + __builtin_ctz(m) : ones_row;
                                m &= m - 1;
                            }
                            uint32_t r[8];
#pragma unroll
                            for (int u = 0; u < 8; ++u) r[u] = col[row[u] * stride];
#pragma unroll
                            for (int u = 0; u < 8; ++u) acc &= r[u];
                        }
                    }
                }
            }
            uint32_t v = active ? (acc >> fg.shift) & fg.mask : 0u;
            if (p.direct) {
                // one or two nodes: the clause against each node's own literal words (kernels.py:443-466 as
                // it stands), lane w on word w; no literal-major rows are read or staged
                uint32_t bits = 0u;
                for (int node = 0; node < n_now; ++node) {
                    bool violated = false;
                    for (int w0 = 0; w0 < LA; w0 += 64) {
                        uint32_t mine = w0 == 0 ? first_words : (w0 + lane < LA ? inc[(w0 + lane) * B] : 0u);
                        if (w0 != 0 && w0 + lane == LA - 1) mine &= p.filter;
                        const uint32_t xs = w0 + lane < LA ? x_now[node * LA + w0 + lane] : 0xFFFFFFFFu;
                        violated |= __ballot((mine & ~xs) != 0) != 0;
                    }
                    if (!violated && (int)types_lds[i & 1][node] == c % p.n_types) bits |= 1u << node;
                }
                v = lane == 0 ? bits : 0u;
            }
            if (filter_only && !all_rows) {
                // lane L holds nodes 32 L .. 32 L + 31: the surviving ones are walked on the scalar unit; lane w
                // compares include word w with the node's literal word w (LDS copy of the graph's X rows)
                unsigned long long live = __ballot(v != 0);
                while (live) {
                    const int L = __ffsll((long long)live) - 1;
                    live &= live - 1;
                    uint32_t word = __builtin_amdgcn_readlane(v, L);
                    uint32_t cleared = 0;
                    while (word) {
                        const int b = __builtin_ctz(word);
                        word &= word - 1;
                        const uint32_t *x = x_now + (L * 32 + b) * LA;
                        bool violated = false;
                        for (int w0 = 0; w0 < LA; w0 += 64) {
                            uint32_t mine = w0 == 0 ? first_words : (w0 + lane < LA ? inc[(w0 + lane) * B] : 0u);
                            if (w0 != 0 && w0 + lane == LA - 1) mine &= p.filter;
                            const uint32_t xs = w0 + lane < LA ? x[w0 + lane] : 0xFFFFFFFFu;
                            violated |= __ballot((mine & ~xs) != 0) != 0;
                        }
                        if (violated) cleared |= 1u << b;
                    }
                    if (lane == L) v &= ~cleared;
                }
            }
            const int pc = __popc(v);
            int true_nodes, before;
            wave_count_scan(pc, lane, &true_nodes, &before);
            bool fired = true_nodes > 0;
            int node = -1;
            if (n_now == 0) {
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
            if (lane == 0) {
                node_of[cl] = node;
                incl_of[cl] = included;
            }
            if (fired)
                for (int k = lane; k < K; k += 64) atomicAdd(&votes[k], wts[cl * K + k]);  // LDS
        }

        // ---- 2. class sums across the device (see the header comment)
        if (tid == 0) go_on = 1;
        lds_barrier();  // the group's votes are complete
        if (tid >= poll0 && tid - poll0 < K) {  // (K <= FITP_BLOCK: one class per thread)
            const int k = tid - poll0;
            __hip_atomic_fetch_add(&slot_now[(k * FITP_SUM_PARTS + (int)(blockIdx.x % FITP_SUM_PARTS)) * FITP_SUM_STRIDE], FITP_ARRIVED + (unsigned long long)(long long)votes[k], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            votes[k] = 0;
        }
        // Work that does not need the class sums is done while the other groups arrive: the next
        // graph's rows, literal words and labels are requested (straight into the other LDS
        // buffers; they are waited for at the end of the step)
        {
            // element at = row * words + w; a thread's elements are FITP_BLOCK apart: step (row, w) without dividing
            const uint32_t *tile = p.tiles + (int64_t)fn.tile * p.tg.rows * p.tg.tw + fn.word0;
            if (fn.words != div_words) {  // the divisions are redone only when the slot width changes
                div_words = fn.words;
                div_dr = loaders / fn.words;
                div_r0 = tid / fn.words;
            }
            const int dr = div_dr, dw = loaders - dr * fn.words;
            int r = div_r0, w = tid - r * fn.words;
            uint32_t *dst = rows_buf[(i + 1) & 1] + wave * 64;
            for (int at0 = 0; at0 < next_total && tid < loaders; at0 += loaders) {
                if (at0 + tid < next_total) fitp_load_to_lds(tile + (int64_t)r * p.tg.tw + w, dst + at0);
                r += dr;
                w += dw;
                if (w >= fn.words) {
                    w -= fn.words;
                    ++r;
                }
            }
        }
        const int next_x_total = has_next ? n_next * LA : 0;
        {
            const uint32_t *src = p.X + (int64_t)base_next * LA + tid;
            uint32_t *dst = x_buf[(i + 1) & 1] + wave * 64;
            for (int at0 = 0; at0 < next_x_total && tid < loaders; at0 += loaders)
                if (at0 + tid < next_x_total) fitp_load_to_lds(src + at0, dst + at0);
        }
        if (has_next) {
            const uint32_t *src = (const uint32_t *)p.encoded_Y + (int64_t)(ex + 1) * K + tid;
            uint32_t *dst = y_buf[(i + 1) & 1] + wave * 64;
            for (int at0 = 0; at0 < K && tid < loaders; at0 += loaders)
                if (at0 + tid < K) fitp_load_to_lds(src + at0, dst + at0);
        }
        if (p.direct && has_next && tid < n_next) types_lds[(i + 1) & 1][tid] = type_ahead;
        // The random words of the feedback gates are drawn by the waves that do not poll, while the
        // class sums are on their way. (Drawing the Type I feedback bits of every (clause, class,
        // word) here as well costs more generator work than the exchange hides: they are drawn
        // afterwards, for the pairs that turn out to need them.)
        const int pollers = (K + 63) & ~63, helpers = FITP_BLOCK - pollers;
        if (helpers >= FITP_BLOCK / 2) {
            // (the polling threads are the first `pollers`, or - set apart - within the last 64)
            if (poll_apart ? tid < poll0 : tid >= pollers)
                for (int j = poll_apart ? tid : tid - pollers; j < n_own * K; j += helpers) {
                    const int cl = j / K, k = j - cl * K;
                    philox_out r = philox4x32_10((uint32_t)(c0 + cl), (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, p.k0, p.k1);
                    gate[2 * j] = r.v[0];
                    gate[2 * j + 1] = r.v[1];
                }
        } else {
            for (int j = tid; j < n_own * K; j += FITP_BLOCK) {
                const int cl = j / K, k = j - cl * K;
                philox_out r = philox4x32_10((uint32_t)(c0 + cl), (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, p.k0, p.k1);
                gate[2 * j] = r.v[0];
                gate[2 * j + 1] = r.v[1];
            }
            lds_barrier();
        }
        if (tid >= poll0 && tid - poll0 < K) {
            const int k = tid - poll0;
            const unsigned long long everyone = (unsigned long long)gridDim.x;
            auto read_sum = [](const unsigned long long *slot, int k) {
                unsigned long long part[FITP_SUM_PARTS], all = 0ull;
#pragma unroll
                for (int s = 0; s < FITP_SUM_PARTS; ++s)
                    part[s] = __hip_atomic_load(&slot[(k * FITP_SUM_PARTS + s) * FITP_SUM_STRIDE], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int s = 0; s < FITP_SUM_PARTS; ++s) all += part[s];
                return all;
            };
            auto arrivals = [](unsigned long long now, unsigned long long before) {
                return ((now - before + FITP_HALF) >> 48) & 0xFFFFull;
            };
            uint32_t *seen_slot = seen + (size_t)(i % 3) * 2 * K;
            const unsigned long long seen_own = ((unsigned long long)seen_slot[K + k] << 32) | seen_slot[k];
            uint32_t polls = 0;
            unsigned long long waiting_since = 0ull;
            unsigned long long word = 0ull;
            bool ok = !p.force_abort;
            if (!ok) __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            while (ok) {
                word = read_sum(slot_now, k);
                if (arrivals(word, seen_own) == everyone) break;
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
            // for the slot's next use, three examples on
            seen_slot[k] = (uint32_t)word, seen_slot[K + k] = (uint32_t)(word >> 32);
        }
        __builtin_amdgcn_s_waitcnt(FITP_WAIT_VMEM);  // the next graph's words are in LDS
        if (tid < 2) after_lds[tid] = after;
        lds_barrier();
        if (!go_on) break;  // uniform over the group; every group leaves at its next check

        // ---- 3. feedback (K8) and automaton updates (K9) on the LDS copies
        const int32_t *y = (const int32_t *)y_buf[i & 1];
        const uint32_t *X_rows = x_now;  // the graph's literal words, node-major, in LDS
        auto decide = [&](int j, int k) {  // K8 for (clause, class) pair j = cl * K + k
            const int cl = j / K;
            int cs = sums[k];
            cs = cs > p.T ? p.T : (cs < -p.T ? -p.T : cs);
            const int yk = y[k];
            const int target = 1 - 2 * (cs > yk);
            int w = wts[j];
            const int sign = (w >= 0) - (w < 0);
            int err = yk - cs;
            err = err < 0 ? -err : err;
            const bool skip = (target == -1 && (uint64_t)gate[2 * j] >= p.q_thr) ||
                              ((uint64_t)gate[2 * j + 1] * (uint64_t)(2 * (int64_t)p.T) >= ((uint64_t)err << 32));
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
            return u;
        };
        if (wave_local) {
            // One clause per wave and few (class, word) pairs per clause: the wave decides for the clause's classes, draws the Type I feedback
            // bits of the (class, word) pairs that need them and updates the clause's automata, with
            // no barrier in between (a wave's LDS accesses are carried out in order).
            if (wave < n_own) {
                const int cl = wave;
                bool any = false;
                for (int k0 = 0; k0 < K; k0 += 64) {
                    const int k = k0 + lane;
                    const int u = k < K ? decide(cl * K + k, k) : 0;
                    any |= __ballot(u != 0) != 0ull;
                    const unsigned long long type1 = __ballot(u > 0);
                    const int n_items = __popcll(type1) * LA;
                    for (int t = lane; t < n_items; t += 64) {
                        const int nth = t / LA, w = t - nth * LA;
                        unsigned long long m = type1;
                        for (int skip = 0; skip < nth; ++skip) m &= m - 1;
                        const int kk = k0 + __ffsll((long long)m) - 1;
                        fbits[((size_t)cl * LA + w) * K + kk] =
                            gtm_feedback_bits(p.k0, p.k1, (uint32_t)(c0 + cl), (uint32_t)w, step, 0u, (uint32_t)kk, p.thr16);
                    }
                }
                fitp_wave_lds_sync();
                if (any) {
                    const int node = node_of[cl];
                    const bool fired = node != -1;
                    const bool within = incl_of[cl] <= p.max_included;
                    for (int w = lane; w < LA; w += 64) {
                        const uint32_t x = fired ? X_rows[node * LA + w] : 0u;
                        feedback_word<MAXB>(ta + ((size_t)cl * LA + w) * B, B, K, upd + cl * K, 1, fired, within, p.boost, x, p.k0,
                                            p.k1, (uint32_t)(c0 + cl), (uint32_t)w, step, 0u, p.thr16,
                                            fbits + ((size_t)cl * LA + w) * K);
                    }
                }
            }
        } else {
            for (int j = tid; j < n_own * K; j += FITP_BLOCK) decide(j, j % K);
            lds_barrier();
            // Type I feedback bits for the (clause, class) pairs that need them: the pairs are listed
            // first (wave 0, ballots), then one thread per (listed pair, word) draws the bits, so that
            // the lanes that run the generator are (nearly) all busy
            if (wave == 0) {
                int n_listed = 0;
                for (int j0 = 0; j0 < n_own * K; j0 += 64) {
                    const int j = j0 + lane;
                    const bool need = j < n_own * K && upd[j] > 0;
                    const unsigned long long m = __ballot(need);
                    if (need) pair_list[n_listed + __popcll(m & ((1ull << lane) - 1ull))] = j;
                    n_listed += __popcll(m);
                }
                if (lane == 0) n_pairs = n_listed;
            }
            lds_barrier();
            for (int t = tid; t < n_pairs * LA; t += FITP_BLOCK) {
                const int j = pair_list[t / LA], w = t % LA;
                const int cl = j / K, k = j - cl * K;
                fbits[((size_t)cl * LA + w) * K + k] =
                    gtm_feedback_bits(p.k0, p.k1, (uint32_t)(c0 + cl), (uint32_t)w, step, 0u, (uint32_t)k, p.thr16);
            }
            lds_barrier();
            for (int j = tid; j < n_own * LA; j += FITP_BLOCK) {
                const int cl = j / LA, w = j - cl * LA;
                const int32_t *u_of = upd + cl * K;
                bool any = false;
                for (int k = 0; k < K; ++k) any |= u_of[k] != 0;
                if (!any) continue;
                const int node = node_of[cl];
                const bool fired = node != -1;
                const bool within = incl_of[cl] <= p.max_included;
                const uint32_t x = fired ? X_rows[node * LA + w] : 0u;
                feedback_word<MAXB>(ta + (size_t)j * B, B, K, u_of, 1, fired, within, p.boost, x, p.k0, p.k1,
                                  (uint32_t)(c0 + cl), (uint32_t)w, step, 0u, p.thr16, fbits + (size_t)j * K);
            }
        }
        // With the feedback inside the clause's wave, the wave goes on to evaluate its clause on the
        // next graph (everything that evaluation reads was complete at the barrier above).
        if (!wave_local) lds_barrier();
        n_now = n_next;
        base_now = base_next;
        n_next = (int)after_lds[0];
        base_next = after_lds[1];
    }
    __builtin_amdgcn_s_waitcnt(FITP_WAIT_VMEM);  // no load into LDS is left in flight when the group ends
    lds_barrier();
    // own state -> global memory (also after an abort: every clause is left as of some whole step)
    for (int i = tid; i < n_own * LA * B; i += FITP_BLOCK) p.bank[(int64_t)c0 * LA * B + i] = ta[i];
    for (int i = tid; i < n_own * K; i += FITP_BLOCK) {
        int cl = i / K, k = i - cl * K;
        p.weights[(int64_t)k * p.C + c0 + cl] = wts[i];
    }
}
