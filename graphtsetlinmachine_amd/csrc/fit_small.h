// A run of training examples (the loop at tm.py:669-747) of a SMALL model with
// message layers on TINY graphs (at most 64 nodes, MESSAGE_SIZE a multiple of
// 32) as one launch of one workgroup: the automata of every bank, the weights
// and everything a step produces live in LDS, and the phases of a step are
// separated by workgroup barriers only.  At this size a step is a chain of
// dependent latencies, not work: 4 + 3 per message layer barriers instead of
// six kernel launches per example.
//
// Per example (one line per barrier-separated phase):
//   layer 0  K1: thread per (clause, node): (include & ~X[node]) == 0 and the
//            node-type gate (kernels.py:443-466); meanwhile the threads at the
//            other end of the block draw the step's random numbers for K7 and K8
//   per message layer
//     send   K3: per-node bit vectors of what the true clauses send
//            (kernels.py:565-588)
//     edges  K4/K5: the vectors rotated along the edges, ORed at the far end
//     K2     thread per (clause, node) against the message bank's include
//            words; the negated message literals are the complement of the
//            received vector (kernels.py:505-527)
//   K7, K6   node pick and class sums (kernels.py:319-354, :279-317)
//   K8       feedback decision, weight update (kernels.py:356-405)
//   K9, K10  Type I / II on every bank (kernels.py:98-242)
// The random numbers are the same counter-based ones as everywhere else, so the
// result equals the other training paths bit for bit.
//
// Memory latency is kept off that chain: the hypervector bits live in LDS, and
// while example i is being worked on the loads of example i + 1 (literal words,
// node types, edge counts and offsets, labels) and of the node count and offset
// of example i + 2 are in flight into registers; they land in the other half of
// double-buffered LDS arrays before the step's last barrier.  The edges of
// example i are fetched at the top of its step and parked in LDS right before
// the first message layer walks them.  The barriers order LDS traffic only, so
// none of them waits for these loads.  LDS loads inside a phase are issued in
// batches (no early exit inside a batch), since one thread's chain of dependent
// LDS round trips is what a phase costs.
#pragma once

constexpr int FITS_BLOCK = 256;
constexpr int FITS_MAX_NODES = 64;
constexpr size_t FITS_MAX_LDS_BYTES = 128 * 1024;  // of the 160 KB a workgroup can have
constexpr int FITS_X_AHEAD = 4;                    // literal words per thread fetched ahead; the rest is read at the step's end
constexpr int FITS_EDGES_LDS = FITS_BLOCK;         // edges of a graph parked in LDS (more: read in place)
constexpr int FITS_Y_LDS = 64;                     // classes whose labels are fetched ahead (K <= this, else read in place)

struct FitSmallParams {
    // data set
    const uint32_t *X, *node_type, *node_index, *n_nodes, *n_edges, *edge_index, *edge;
    const int32_t *encoded_Y;
    int first_example, n_examples;
    uint32_t first_step;
    int n_types, has_edges;
    // model
    uint32_t *bank[GTM_MAX_DEPTH];     // bank 0: literals of the nodes; bank l: message literals of layer l
    uint32_t filter[GTM_MAX_DEPTH];    // valid bits of a bank's last include word
    uint32_t thr16[GTM_MAX_DEPTH];
    int32_t *weights;                  // [K][C]
    const uint32_t *hv;                // [C][MB]
    int depth, C, LA, MC, MW, MB, B, K, T, negative, boost, max_included;
    uint32_t k0, k1;
    uint64_t q_thr;
};

// LDS words the kernel needs (the host checks it against the limit it sets).
inline size_t fit_small_lds_words(int depth, int C, int LA, int MC, int MW, int MB, int B, int K) {
    const size_t banks = (size_t)C * (LA + (size_t)(depth - 1) * MC) * B;
    return banks + (size_t)K * C                              // weights
           + (size_t)C * MB                                   // hypervector bits
           + 2 * ((size_t)FITS_MAX_NODES * LA + 3 * FITS_MAX_NODES + FITS_Y_LDS + 2)  // graph data, two examples
           + 2 * (size_t)FITS_EDGES_LDS                       // edges
           + 2 * (size_t)C * 2                                // truth of two layers, 2 words per clause
           + (size_t)depth * FITS_MAX_NODES * MW              // sent; got per layer
           + (size_t)K + 2 * (size_t)C + (size_t)C * K        // class sums, picked node, include count, updates
           + (size_t)C + 2 * (size_t)C * K;                   // random draws of K7 and K8
}

// AND over a run of include words (stride B apart, top bit plane) against literal words:
// returns the violated bits ORed together, adds the number of included literals.
__device__ __forceinline__ uint32_t fits_violations(const uint32_t *inc, int B, const uint32_t *x, int n_words,
                                                     bool negated, uint32_t last_filter, int *included) {
    uint32_t bad = 0u;
    int count = 0;
    int w = 0;
    for (; w + 4 <= n_words; w += 4) {
        uint32_t i0 = inc[(w + 0) * B], i1 = inc[(w + 1) * B], i2 = inc[(w + 2) * B], i3 = inc[(w + 3) * B];
        uint32_t x0 = x[w + 0], x1 = x[w + 1], x2 = x[w + 2], x3 = x[w + 3];
        if (w + 4 == n_words) i3 &= last_filter;
        if (negated) x0 = ~x0, x1 = ~x1, x2 = ~x2, x3 = ~x3;
        bad |= (i0 & ~x0) | (i1 & ~x1) | (i2 & ~x2) | (i3 & ~x3);
        count += __popc(i0) + __popc(i1) + __popc(i2) + __popc(i3);
    }
    for (; w < n_words; ++w) {
        uint32_t i0 = inc[w * B], x0 = x[w];
        if (w + 1 == n_words) i0 &= last_filter;
        if (negated) x0 = ~x0;
        bad |= i0 & ~x0;
        count += __popc(i0);
    }
    *included += count;
    return bad;
}

__global__ __launch_bounds__(FITS_BLOCK) void k_fit_small(FitSmallParams p) {
    extern __shared__ __align__(16) uint32_t lds[];
    const int tid = threadIdx.x;
    const int C = p.C, LA = p.LA, MC = p.MC, MW = p.MW, B = p.B, K = p.K, layers = p.depth - 1;

    // LDS carve-up: bank 0, then the message banks (all of one size), then the rest
    const size_t bank0_words = (size_t)C * LA * B, message_bank_words = (size_t)C * MC * B;
    auto bank_of = [&](int l) { return l == 0 ? lds : lds + bank0_words + (size_t)(l - 1) * message_bank_words; };
    int32_t *wts = (int32_t *)(lds + bank0_words + (size_t)layers * message_bank_words);  // [K][C]
    uint32_t *hv = (uint32_t *)(wts + K * C);      // [C][MB]
    // per example, double-buffered: literal words [nodes][LA]; node type, edge count, first edge
    // [3][nodes]; labels [FITS_Y_LDS]; node count and first node of the example after
    const int graph_words = FITS_MAX_NODES * LA + 3 * FITS_MAX_NODES + FITS_Y_LDS + 2;
    uint32_t *graph_buf = hv + C * p.MB;
    uint32_t *edges_lds = graph_buf + 2 * graph_words;  // [FITS_EDGES_LDS][2]
    uint32_t *truth[2] = {edges_lds + 2 * FITS_EDGES_LDS, edges_lds + 2 * FITS_EDGES_LDS + 2 * C};  // [C][2]
    uint32_t *sent = truth[1] + 2 * C;             // [nodes][MW]
    uint32_t *got_all = sent + FITS_MAX_NODES * MW;  // [layers][nodes][MW]: what each node received, per layer
    int32_t *sums = (int32_t *)(got_all + (size_t)layers * FITS_MAX_NODES * MW);  // [K]
    int32_t *node_of = sums + K;                   // [C]
    int32_t *incl_of = node_of + C;                // [C]
    int32_t *upd = incl_of + C;                    // [C][K]
    uint32_t *draw_node = (uint32_t *)(upd + C * K);  // [C]
    uint32_t *draw_update = draw_node + C;         // [C][K][2]

    // state -> LDS
    for (int l = 0; l < p.depth; ++l) {
        uint32_t *dst = bank_of(l);
        const uint32_t *src = p.bank[l];
        for (int i = tid; i < C * (l == 0 ? LA : MC) * B; i += FITS_BLOCK) dst[i] = src[i];
    }
    for (int i = tid; i < K * C; i += FITS_BLOCK) wts[i] = p.weights[i];
    for (int i = tid; i < C * p.MB; i += FITS_BLOCK) hv[i] = p.hv[i];
    for (int i = tid; i < 2 * C; i += FITS_BLOCK) truth[0][i] = 0u;
    for (int i = tid; i < FITS_MAX_NODES * MW; i += FITS_BLOCK) sent[i] = 0u;

    // the first example's data, and the second's node count and offset
    int n_nodes = (int)p.n_nodes[p.first_example];
    {
        const int64_t base = p.node_index[p.first_example];
        uint32_t *x_rows = graph_buf, *field = x_rows + FITS_MAX_NODES * LA, *labels = field + 3 * FITS_MAX_NODES;
        for (int j = tid; j < n_nodes * LA; j += FITS_BLOCK) x_rows[j] = p.X[base * LA + j];
        for (int j = tid; j < n_nodes; j += FITS_BLOCK) {
            field[j] = p.node_type[base + j];
            field[FITS_MAX_NODES + j] = p.has_edges ? p.n_edges[base + j] : 0u;
            field[2 * FITS_MAX_NODES + j] = p.has_edges ? p.edge_index[base + j] : 0u;
        }
        for (int k = tid; k < K && k < FITS_Y_LDS; k += FITS_BLOCK)
            labels[k] = (uint32_t)p.encoded_Y[(int64_t)p.first_example * K + k];
        if (tid < 2 && p.n_examples > 1)
            labels[FITS_Y_LDS + tid] = (tid == 0 ? p.n_nodes : p.node_index)[p.first_example + 1];
    }
    lds_barrier();

    for (int i = 0; i < p.n_examples; ++i) {
        const int ex = p.first_example + i;
        const uint32_t step = p.first_step + (uint32_t)i;
        const int nn = n_nodes > 0 ? n_nodes : 1;  // a graph without nodes: one stand-in pair per clause
        uint32_t *x_rows = graph_buf + (i & 1) * graph_words, *types = x_rows + FITS_MAX_NODES * LA;
        const uint32_t *ne_lds = types + FITS_MAX_NODES, *ei_lds = types + 2 * FITS_MAX_NODES;
        const int32_t *y = (const int32_t *)(types + 3 * FITS_MAX_NODES);
        const uint32_t *header = types + 3 * FITS_MAX_NODES + FITS_Y_LDS;
        uint32_t *x_next = graph_buf + ((i + 1) & 1) * graph_words, *field_next = x_next + FITS_MAX_NODES * LA;

        // ---- loads that land later: example i + 1 (its node count and offset came with example i),
        // the header of example i + 2, the edges of this example
        const bool more = i + 1 < p.n_examples;
        const int n_next = more ? __builtin_amdgcn_readfirstlane((int)header[0]) : 0;
        const int64_t base_next = more ? (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)header[1]) : 0;
        uint32_t x_ahead[FITS_X_AHEAD];
#pragma unroll
        for (int r = 0; r < FITS_X_AHEAD; ++r) {
            const int j = tid + r * FITS_BLOCK;
            x_ahead[r] = j < n_next * LA ? p.X[base_next * LA + j] : 0u;
        }
        uint32_t field_ahead = 0u;
        {
            const int which = tid >> 6, j = tid & 63;
            if (which < 3) {
                if (j < n_next && (which == 0 || p.has_edges))
                    field_ahead = (which == 0 ? p.node_type : which == 1 ? p.n_edges : p.edge_index)[base_next + j];
            } else if (more && j < K) {
                field_ahead = (uint32_t)p.encoded_Y[(int64_t)(ex + 1) * K + j];
            }
        }
        uint32_t header_ahead = 0u;
        if (tid < 2 && i + 2 < p.n_examples) header_ahead = (tid == 0 ? p.n_nodes : p.node_index)[ex + 2];
        int64_t first_edge = 0;
        int graph_edges = 0;
        if (p.has_edges && n_nodes > 0) {
            first_edge = ei_lds[0];
            graph_edges = (int)(ei_lds[n_nodes - 1] + ne_lds[n_nodes - 1] - (uint32_t)first_edge);
        }
        const bool edges_parked = graph_edges <= FITS_EDGES_LDS;
        uint2 edge_ahead = make_uint2(0u, 0u);
        if (edges_parked && tid < graph_edges) edge_ahead = ((const uint2 *)p.edge)[first_edge + tid];

        for (int k = tid; k < K; k += FITS_BLOCK) sums[k] = 0;
        for (int j = tid; j < layers * FITS_MAX_NODES * MW; j += FITS_BLOCK) got_all[j] = 0u;

        // ---- layer 0 (K1), one thread per (clause, node); truth[0] is all zero here
        uint32_t *cur = truth[0], *nxt = truth[1];
        for (int j = tid; j < C * nn; j += FITS_BLOCK) {
            const int c = j / nn, n = j - c * nn;
            const bool match = n_nodes > 0 && (int)types[n] == c % p.n_types;
            if (match || n == 0) {
                int included = 0;
                const uint32_t bad =
                    fits_violations(lds + (size_t)c * LA * B + (B - 1), B, x_rows + n * LA, LA, false, p.filter[0], &included);
                if (n == 0) incl_of[c] = included;
                // a graph without nodes: the reference's arithmetic leaves every clause true (kernels.py:289-295)
                if (n_nodes == 0)
                    cur[2 * c] = 0xFFFFFFFFu;
                else if (match && bad == 0u)
                    atomicOr(&cur[2 * c + (n >> 5)], 1u << (n & 31));
            }
        }
        // the step's random numbers for the node pick (K7) and the feedback decision (K8), drawn
        // from the other end of the block so that they overlap the evaluation when pairs are few
        for (int j = FITS_BLOCK - 1 - tid; j < C + C * K; j += FITS_BLOCK) {
            if (j < C) {
                draw_node[j] = philox4x32_10((uint32_t)j, 0u, step, GTM_TAG_CLAUSE_NODE, p.k0, p.k1).v[0];
            } else {
                const int ck = j - C, c = ck / K, k = ck - c * K;
                philox_out r = philox4x32_10((uint32_t)c, (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, p.k0, p.k1);
                draw_update[2 * ck] = r.v[0];
                draw_update[2 * ck + 1] = r.v[1];
            }
        }
        lds_barrier();

        // ---- message layers; sent is all zero at the start of each
        for (int l = 0; l < layers; ++l) {
            uint32_t *got = got_all + (size_t)l * FITS_MAX_NODES * MW;
            // what each node sends: the hypervector bits of the clauses true at it
            for (int j = tid; j < 2 * C; j += FITS_BLOCK) nxt[j] = 0u;
            for (int j = tid; j < C * n_nodes; j += FITS_BLOCK) {
                const int c = j / n_nodes, n = j - c * n_nodes;
                if ((cur[2 * c + (n >> 5)] >> (n & 31)) & 1u)
                    for (int b = 0; b < p.MB; ++b) {
                        const uint32_t h = hv[c * p.MB + b];
                        atomicOr(&sent[n * MW + (h >> 5)], 1u << (h & 31));
                    }
            }
            // the edges requested at the top of the step are parked here, as late as their first use allows
            if (l == 0 && edges_parked && tid < graph_edges) {
                edges_lds[2 * tid] = edge_ahead.x;
                edges_lds[2 * tid + 1] = edge_ahead.y;
            }
            lds_barrier();
            // along every edge: the vector rotated by the edge type (bit p of the result is bit (p - type) mod M)
            if (graph_edges > 0)
                for (int j = tid; j < n_nodes * MW; j += FITS_BLOCK) {
                    const int n = j / MW, jw = j - n * MW;
                    const uint32_t ne = ne_lds[n];
                    const uint32_t *v = sent + n * MW;
                    for (uint32_t e = 0; e < ne; ++e) {
                        uint32_t dst, type;
                        if (edges_parked) {
                            const uint32_t at = ei_lds[n] - (uint32_t)first_edge + e;
                            dst = edges_lds[2 * at];
                            type = edges_lds[2 * at + 1];
                        } else {
                            dst = p.edge[((int64_t)ei_lds[n] + e) * 2];
                            type = p.edge[((int64_t)ei_lds[n] + e) * 2 + 1];
                        }
                        const uint32_t shift = type % (uint32_t)(MW * 32);
                        const int q = (int)(shift >> 5), r = (int)(shift & 31u);
                        const int a = (jw - q + MW) % MW, below = (a - 1 + MW) % MW;
                        const uint32_t word = r ? (v[a] << r) | (v[below] >> (32 - r)) : v[a];
                        if (word) atomicOr(&got[dst * MW + jw], word);
                    }
                }
            lds_barrier();
            // K2, one thread per (clause, node): include words 0 .. MW - 1 against the received
            // vector, MW .. 2 MW - 1 against its complement
            for (int j = tid; j < FITS_MAX_NODES * MW; j += FITS_BLOCK) sent[j] = 0u;
            for (int j = tid; j < C * nn; j += FITS_BLOCK) {
                const int c = j / nn, n = j - c * nn;
                const bool alive = n_nodes > 0 && ((cur[2 * c + (n >> 5)] >> (n & 31)) & 1u);
                if (alive || n == 0) {
                    const uint32_t *inc = bank_of(l + 1) + (size_t)c * MC * B + (B - 1);
                    int included = 0;
                    uint32_t bad = fits_violations(inc, B, got + n * MW, MW, false, 0xFFFFFFFFu, &included);
                    bad |= fits_violations(inc + (size_t)MW * B, B, got + n * MW, MW, true, p.filter[l + 1], &included);
                    if (n == 0) incl_of[c] += included;
                    if (n_nodes == 0)
                        nxt[2 * c] = 0xFFFFFFFFu;
                    else if (alive && bad == 0u)
                        atomicOr(&nxt[2 * c + (n >> 5)], 1u << (n & 31));
                }
            }
            lds_barrier();
            uint32_t *swap = cur;
            cur = nxt;
            nxt = swap;
        }

        // ---- K7 + K6: node pick and class sums, one thread per clause
        for (int c = tid; c < C; c += FITS_BLOCK) {
            const uint32_t lo = cur[2 * c], hi = cur[2 * c + 1];
            int node = -1;
            bool fired;
            if (n_nodes == 0) {
                fired = true;
            } else {
                const int count = __popc(lo) + __popc(hi);
                fired = count > 0;
                if (fired) {
                    int pick = (int)(((uint64_t)draw_node[c] * (uint64_t)count) >> 32);
                    unsigned long long bits = ((unsigned long long)hi << 32) | lo;
                    for (int j = 0; j < pick; ++j) bits &= bits - 1;
                    node = __ffsll((long long)bits) - 1;
                }
            }
            node_of[c] = node;
            if (fired)
                for (int k = 0; k < K; ++k) atomicAdd(&sums[k], wts[k * C + c]);
        }
        lds_barrier();

        // ---- K8: feedback decision and weight update, one thread per (clause, class)
        const int32_t *y_global = p.encoded_Y + (int64_t)ex * K;
        for (int j = tid; j < 2 * C; j += FITS_BLOCK) truth[0][j] = 0u;  // for the next example's layer 0
        for (int j = tid; j < C * K; j += FITS_BLOCK) {
            const int c = j / K, k = j - c * K;
            int cs = sums[k];
            cs = cs > p.T ? p.T : (cs < -p.T ? -p.T : cs);
            const int yk = K <= FITS_Y_LDS ? y[k] : y_global[k];
            const int target = 1 - 2 * (cs > yk);
            int w = wts[k * C + c];
            const int sign = (w >= 0) - (w < 0);
            int err = yk - cs;
            err = err < 0 ? -err : err;
            const uint32_t r0 = draw_update[2 * j], r1 = draw_update[2 * j + 1];
            const bool skip = (target == -1 && (uint64_t)r0 >= p.q_thr) ||
                              ((uint64_t)r1 * (uint64_t)(2 * (int64_t)p.T) >= ((uint64_t)err << 32));
            const int u = skip ? 0 : target * sign;
            const bool fired = node_of[c] != -1;
            if (u > 0 && fired && (w < 0 ? -(int64_t)w : (int64_t)w) < 2147483647) {
                wts[k * C + c] = w + sign;
            } else if (u < 0 && fired) {
                w -= sign;
                if (p.negative == 0 && w < 1) w = 1;
                wts[k * C + c] = w;
            }
            upd[j] = u;
        }
        lds_barrier();

        // ---- K9, K10: one thread per (clause, automaton word of any bank)
        const int per_clause = LA + layers * MC;
        for (int j = tid; j < C * per_clause; j += FITS_BLOCK) {
            const int c = j / per_clause;
            int w = j - c * per_clause;
            const int32_t *u_of = upd + c * K;
            bool any = false;
            for (int k = 0; k < K; ++k) any |= u_of[k] != 0;
            if (!any) continue;
            const int l = w < LA ? 0 : 1 + (w - LA) / MC;
            if (l > 0) w = (w - LA) - (l - 1) * MC;
            const int chunks = l == 0 ? LA : MC;
            const int node = node_of[c];
            const bool fired = node != -1;
            const bool within = incl_of[c] <= p.max_included;
            uint32_t x = 0u;
            if (fired) {
                if (l == 0) {
                    x = x_rows[node * LA + w];
                } else {
                    const uint32_t *got = got_all + (size_t)(l - 1) * FITS_MAX_NODES * MW + node * MW;
                    x = w < MW ? got[w] : ~got[w - MW];
                }
            }
            uint32_t thr16 = p.thr16[0];
#pragma unroll
            for (int t = 1; t < GTM_MAX_DEPTH; ++t)
                if (t == l) thr16 = p.thr16[t];
            feedback_word_any(bank_of(l) + ((size_t)c * chunks + w) * B, B, K, u_of, 1, fired, within, p.boost, x, p.k0, p.k1,
                              (uint32_t)c, (uint32_t)w, step, (uint32_t)l, thr16);
        }

        // ---- example i + 1 lands in the other buffer
#pragma unroll
        for (int r = 0; r < FITS_X_AHEAD; ++r) {
            const int j = tid + r * FITS_BLOCK;
            if (j < n_next * LA) x_next[j] = x_ahead[r];
        }
        for (int j = tid + FITS_X_AHEAD * FITS_BLOCK; j < n_next * LA; j += FITS_BLOCK) x_next[j] = p.X[base_next * LA + j];
        static_assert(3 * FITS_MAX_NODES + FITS_Y_LDS == FITS_BLOCK, "one thread per word of the node fields and labels");
        field_next[tid] = field_ahead;
        if (tid < 2) field_next[3 * FITS_MAX_NODES + FITS_Y_LDS + tid] = header_ahead;
        n_nodes = n_next;
        lds_barrier();
    }

    // state -> global memory
    for (int l = 0; l < p.depth; ++l) {
        const uint32_t *src = bank_of(l);
        uint32_t *dst = p.bank[l];
        for (int i = tid; i < C * (l == 0 ? LA : MC) * B; i += FITS_BLOCK) dst[i] = src[i];
    }
    for (int i = tid; i < K * C; i += FITS_BLOCK) p.weights[i] = wts[i];
}
