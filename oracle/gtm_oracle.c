/* CPU restatement in plain C of the Graph Tsetlin Machine's hot path.
 *
 * TEST INFRASTRUCTURE ONLY: nothing in the shipped package links or loads this
 * file.  It is a second, independent checker next to oracle/gtm_oracle.py (the
 * two are compared with each other in tests/test_oracle_c.py) and the CPU
 * baseline that bench.py times beside the GPU: inference (gtmc_score) and
 * training (gtmc_fit).
 *
 * It follows the reference's CUDA kernels loop for loop, one graph at a time,
 * on the reference's own memory layouts:
 *   K1  calculate_messages              GraphTsetlinMachine/kernels.py:407-468
 *   K2  calculate_messages_conditional  kernels.py:470-530
 *   K3  prepare_messages                kernels.py:532-547
 *   K4  exchange_messages               kernels.py:549-590
 *   K5  encode_messages                 kernels.py:592-615
 *   K6  evaluate                        kernels.py:279-317
 * sequenced as the reference's driver does (tm.py:563-662, :786-812).  The
 * only liberties are the ones a CPU wants and that cannot change a result: a
 * node's test stops at its first violated word, and graphs are spread over
 * OpenMP threads (they are independent).
 *
 * Layouts: ta_state uint32 [CLAUSES][chunks][STATE_BITS], plane STATE_BITS-1 is
 * the include mask; X uint32 [nodes][LA_CHUNKS]; clause/node bitmap uint32
 * [CLAUSES][NODE_CHUNKS]; edge uint32 [edges][2] = (destination, type);
 * clause_weights int32 [CLASSES][CLAUSES]; hypervectors uint32
 * [CLAUSES][MESSAGE_BITS].
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct {
    int32_t classes, clauses, literals, state_bits, max_nodes, message_size, message_bits, depth;
} gtmc_config;

typedef struct {
    const uint32_t *X, *node_type, *number_of_graph_node_edges, *edge, *node_index, *edge_index, *number_of_graph_nodes;
    int32_t number_of_node_types;
} gtmc_graphs;

static uint32_t tail_filter(int bits) { /* kernels.py:37-47 */
    int r = bits % 32;
    return r == 0 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << r);
}

static int chunks_of(int bits) { return (bits - 1) / 32 + 1; }

/* K1 and K2 share their body: the truth of every clause at every node against a bank's include
 * plane and the nodes' literal words; K2 ANDs the previous layer's bitmap in. */
static void clause_node_bits(int clauses, int node_chunks, int chunks, int state_bits, uint32_t filter,
                             const uint32_t *bank, const uint32_t *node_type, int n_types, int n_nodes,
                             const uint32_t *literal_words, const uint32_t *condition, uint32_t *out) {
    const int n_chunks = (n_nodes - 1) / 32 + 1; /* C division: 1 for a graph without nodes */
    const uint32_t node_filter = n_nodes % 32 != 0 ? ~(0xFFFFFFFFu << (n_nodes % 32)) : 0xFFFFFFFFu;
#pragma omp parallel for schedule(static) /* (serial inside gtmc_score's own parallel region) */
    for (int clause = 0; clause < clauses; ++clause) {
        const uint32_t *ta = bank + (size_t)clause * chunks * state_bits + (state_bits - 1);
        for (int node_chunk = 0; node_chunk < node_chunks; ++node_chunk) {
            uint32_t word = ~0u;
            for (int pos = 0; pos < 32 && node_chunk * 32 + pos < n_nodes; ++pos) {
                const int node = node_chunk * 32 + pos;
                int holds = (int)node_type[node] == clause % n_types;
                const uint32_t *x = literal_words + (size_t)node * chunks;
                for (int w = 0; holds && w < chunks; ++w) {
                    const uint32_t include = w == chunks - 1 ? ta[(size_t)w * state_bits] & filter : ta[(size_t)w * state_bits];
                    if ((include & x[w]) != include) holds = 0;
                }
                if (!holds) word &= ~(1u << pos);
            }
            if (node_chunk == n_chunks - 1) word &= node_filter;
            if (condition) word &= condition[(size_t)clause * node_chunks + node_chunk];
            out[(size_t)clause * node_chunks + node_chunk] = word;
        }
    }
}

/* K3 + K4 + K5: the packed message literals of every node, [n_nodes][message_chunks]. */
static void build_messages(const gtmc_config *cfg, int node_chunks, int n_nodes, const uint32_t *hypervectors,
                           const uint32_t *bitmap, const uint32_t *n_edges, const uint32_t *edge, uint8_t *x_int,
                           uint32_t *packed) {
    const int M = cfg->message_size, literals = 2 * M, chunks = chunks_of(literals);
    for (int node = 0; node < n_nodes; ++node) { /* K3 */
        memset(x_int + (size_t)node * literals, 0, (size_t)M);
        memset(x_int + (size_t)node * literals + M, 1, (size_t)M);
    }
    for (int clause = 0; clause < cfg->clauses; ++clause) { /* K4 */
        const uint32_t *bits = hypervectors + (size_t)clause * cfg->message_bits;
        size_t at = 0; /* first out-edge of the source node, relative to the graph's first edge */
        for (int source = 0; source < n_nodes; ++source) {
            if (bitmap[(size_t)clause * node_chunks + source / 32] & (1u << (source % 32)))
                for (uint32_t i = 0; i < n_edges[source]; ++i) {
                    const uint32_t destination = edge[(at + i) * 2], type = edge[(at + i) * 2 + 1];
                    for (int b = 0; b < cfg->message_bits; ++b) {
                        const uint32_t shifted = (bits[b] + type) % (uint32_t)M;
                        x_int[(size_t)destination * literals + shifted] = 1;
                        x_int[(size_t)destination * literals + M + shifted] = 0;
                    }
                }
            at += n_edges[source];
        }
    }
    for (int node = 0; node < n_nodes; ++node) /* K5 */
        for (int chunk = 0; chunk < chunks; ++chunk) {
            uint32_t message = 0;
            for (int pos = 0; pos < 32 && chunk * 32 + pos < literals; ++pos)
                if (x_int[(size_t)node * literals + chunk * 32 + pos]) message |= 1u << pos;
            packed[(size_t)node * chunks + chunk] = message;
        }
}

/* K6: unclipped votes per class. */
static void class_sums(const gtmc_config *cfg, int node_chunks, int n_nodes, const uint32_t *bitmap,
                       const int32_t *weights, int32_t *sums) {
    const int n_chunks = (n_nodes - 1) / 32 + 1;
    const uint32_t node_filter = n_nodes % 32 != 0 ? ~(0xFFFFFFFFu << (n_nodes % 32)) : 0xFFFFFFFFu;
    for (int k = 0; k < cfg->classes; ++k) sums[k] = 0;
    for (int clause = 0; clause < cfg->clauses; ++clause) {
        const uint32_t *row = bitmap + (size_t)clause * node_chunks;
        int fired = 0;
        for (int w = 0; w < n_chunks - 1 && !fired; ++w) fired = row[w] != 0;
        if (row[n_chunks - 1] & node_filter) fired = 1;
        if (fired)
            for (int k = 0; k < cfg->classes; ++k) sums[k] += weights[(size_t)k * cfg->clauses + clause];
    }
}

/* Class sums of the graphs graph_ids[0..n) (tm.py:786-812).  message_ta_state: depth - 1 banks.
 * Returns 0, or -1 when memory runs out. */
int gtmc_score(const gtmc_config *cfg, const gtmc_graphs *g, const uint32_t *ta_state,
               const uint32_t *const *message_ta_state, const int32_t *clause_weights, const uint32_t *hypervectors,
               const int32_t *graph_ids, int32_t n, int32_t threads, int32_t *sums_out) {
    const int la_chunks = chunks_of(cfg->literals), message_chunks = chunks_of(2 * cfg->message_size);
    const int node_chunks = chunks_of(cfg->max_nodes > 0 ? cfg->max_nodes : 1);
    const uint32_t filter = tail_filter(cfg->literals), message_filter = tail_filter(2 * cfg->message_size);
    int failed = 0;
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#else
    (void)threads;
#endif
#pragma omp parallel
    {
        const size_t bitmap_words = (size_t)cfg->clauses * node_chunks;
        const size_t nodes = (size_t)(cfg->max_nodes > 0 ? cfg->max_nodes : 1);
        uint32_t *bitmap_a = malloc(bitmap_words * 4), *bitmap_b = malloc(bitmap_words * 4);
        uint8_t *x_int = cfg->depth > 1 ? malloc(nodes * 2 * (size_t)cfg->message_size) : NULL;
        uint32_t *packed = cfg->depth > 1 ? malloc(nodes * message_chunks * 4) : NULL;
        if (!bitmap_a || !bitmap_b || (cfg->depth > 1 && (!x_int || !packed))) {
#pragma omp atomic write
            failed = 1;
        }
#pragma omp barrier
        if (!failed) { /* the same on every thread after the barrier */
#pragma omp for schedule(dynamic, 16)
            for (int32_t i = 0; i < n; ++i) {
                const int32_t e = graph_ids[i];
                const int n_nodes = (int)g->number_of_graph_nodes[e];
                const size_t base = g->node_index[e];
                const uint32_t *types = g->node_type + base;
                uint32_t *now = bitmap_a, *next = bitmap_b;
                clause_node_bits(cfg->clauses, node_chunks, la_chunks, cfg->state_bits, filter, ta_state, types,
                                 g->number_of_node_types, n_nodes, g->X + base * la_chunks, NULL, now);
                for (int layer = 0; layer + 1 < cfg->depth; ++layer) {
                    const uint32_t *n_edges = g->number_of_graph_node_edges + base;
                    const uint32_t *edges = n_nodes > 0 ? g->edge + (size_t)g->edge_index[base] * 2 : g->edge;
                    build_messages(cfg, node_chunks, n_nodes, hypervectors, now, n_edges, edges, x_int, packed);
                    clause_node_bits(cfg->clauses, node_chunks, message_chunks, cfg->state_bits, message_filter,
                                     message_ta_state[layer], types, g->number_of_node_types, n_nodes, packed, now, next);
                    uint32_t *swap = now;
                    now = next;
                    next = swap;
                }
                class_sums(cfg, node_chunks, n_nodes, now, clause_weights, sums_out + (size_t)i * cfg->classes);
            }
        }
        free(bitmap_a);
        free(bitmap_b);
        free(x_int);
        free(packed);
    }
    return failed ? -1 : 0;
}

/* ---------------------------------------------------------------------------
 * Training (tm.py:664-752): K7 select_clause_node (kernels.py:319-354), K8
 * select_clause_updates (kernels.py:356-405), K9/K10 update and update_message
 * (kernels.py:55-242), one example after the other.  The random numbers are the
 * counter-based Philox4x32-10 ones that the NumPy oracle and the HIP kernels
 * share (the reference's cuRAND stream depends on its launch shape and cannot be
 * restated): which counter feeds which decision is stated at each use. */

enum { TAG_CLAUSE_NODE = 2, TAG_CLAUSE_UPDATES = 3, TAG_FEEDBACK = 4 };

static void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t out[4]) {
    for (int round = 0; round < 10; ++round) { /* Salmon et al., SC'11; Random123 philox.h */
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1,
                       n3 = (uint32_t)p0;
        c0 = n0, c1 = n1, c2 = n2, c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

typedef struct {
    int32_t threshold, boost_true_positive_feedback, max_included_literals, negative_clauses;
    uint64_t q_threshold;   /* a negative target is kept when its 32-bit draw is below this */
    uint64_t seed;
    uint32_t feedback_threshold[8]; /* per bank: a Type I bit is set when its 16-bit draw is below this */
} gtmc_training;

/* kernels.py:55-74 / :77-96 on one word of automata: saturating +1 / -1 on the automata in `active`. */
static void inc_word(uint32_t *ta, int state_bits, uint32_t active) {
    uint32_t carry = active;
    for (int b = 0; b < state_bits; ++b) {
        const uint32_t next = ta[b] & carry;
        ta[b] ^= carry;
        carry = next;
    }
    for (int b = 0; b < state_bits; ++b) ta[b] |= carry;
}

static void dec_word(uint32_t *ta, int state_bits, uint32_t active) {
    uint32_t carry = active;
    for (int b = 0; b < state_bits; ++b) {
        const uint32_t next = ~ta[b] & carry;
        ta[b] ^= carry;
        carry = next;
    }
    for (int b = 0; b < state_bits; ++b) ta[b] &= ~carry;
}

/* The 32 Type I feedback bits of word `w` of clause `c` for one class: four Philox blocks at
 * counters (c, 4 w + j, step, TAG_FEEDBACK | bank << 8 | class << 16); bit b takes block b / 8,
 * output word (b % 8) / 2, its low half for even b and its high half for odd b. */
static uint32_t feedback_bits(const gtmc_training *t, uint32_t step, int bank, int class_id, int c, int w) {
    const uint32_t k0 = (uint32_t)t->seed, k1 = (uint32_t)(t->seed >> 32);
    const uint32_t c3 = (uint32_t)TAG_FEEDBACK | ((uint32_t)bank << 8) | ((uint32_t)class_id << 16);
    uint32_t bits = 0;
    for (int j = 0; j < 4; ++j) {
        uint32_t r[4];
        philox4x32_10((uint32_t)c, (uint32_t)(4 * w + j), step, c3, k0, k1, r);
        for (int q = 0; q < 8; ++q) {
            const uint32_t half = (q & 1) ? r[q >> 1] >> 16 : r[q >> 1] & 0xFFFFu;
            if (half < t->feedback_threshold[bank]) bits |= 1u << (8 * j + q);
        }
    }
    return bits;
}

/* K9 / K10 for one bank: classes in ascending order on the same automata (kernels.py:205-207, 236-238). */
static void feedback(const gtmc_config *cfg, const gtmc_training *t, uint32_t step, int bank_id, uint32_t *bank,
                     int chunks, const int32_t *clause_node, const int32_t *n_incl, const uint32_t *literal_words,
                     const int32_t *updates) {
    const int B = cfg->state_bits;
#pragma omp parallel for schedule(static)
    for (int c = 0; c < cfg->clauses; ++c) {
        const int fired = clause_node[c] != -1;
        const int within = n_incl[c] <= t->max_included_literals;
        for (int w = 0; w < chunks; ++w) {
            uint32_t *ta = bank + ((size_t)c * chunks + w) * B;
            const uint32_t x = fired ? literal_words[(size_t)clause_node[c] * chunks + w] : 0u;
            for (int k = 0; k < cfg->classes; ++k) {
                const int32_t u = updates[(size_t)k * cfg->clauses + c];
                if (u > 0) {
                    const uint32_t fb = feedback_bits(t, step, bank_id, k, c, w);
                    if (fired && within) {
                        inc_word(ta, B, t->boost_true_positive_feedback == 1 ? x : x & ~fb);
                        dec_word(ta, B, ~x & fb);
                    } else {
                        dec_word(ta, B, fb);
                    }
                } else if (u < 0 && fired) {
                    inc_word(ta, B, ~x & ~ta[B - 1]);
                }
            }
        }
    }
}

static int include_count(const uint32_t *bank, int clause, int chunks, int state_bits, uint32_t filter) {
    int n = 0; /* kernels.py:244-277 */
    for (int w = 0; w < chunks; ++w) {
        uint32_t include = bank[((size_t)clause * chunks + w) * state_bits + state_bits - 1];
        if (w == chunks - 1) include &= filter;
        n += __builtin_popcount(include);
    }
    return n;
}

/* One pass over the examples graph_ids[0..n) in that order; example i is training step
 * first_step + i.  encoded_Y is [graphs][classes] (+T / -T, tm.py:949-951).  The banks and the
 * weights are updated in place.  Returns 0, or -1 when memory runs out. */
int gtmc_fit(const gtmc_config *cfg, const gtmc_training *t, const gtmc_graphs *g, uint32_t *ta_state,
             uint32_t *const *message_ta_state, int32_t *clause_weights, const uint32_t *hypervectors,
             const int32_t *encoded_Y, const int32_t *graph_ids, int32_t n, uint64_t first_step, int32_t threads) {
    const int la_chunks = chunks_of(cfg->literals), message_chunks = chunks_of(2 * cfg->message_size);
    const int node_chunks = chunks_of(cfg->max_nodes > 0 ? cfg->max_nodes : 1);
    const uint32_t filter = tail_filter(cfg->literals), message_filter = tail_filter(2 * cfg->message_size);
    const uint32_t k0 = (uint32_t)t->seed, k1 = (uint32_t)(t->seed >> 32);
    const int C = cfg->clauses, K = cfg->classes, T = t->threshold, layers = cfg->depth - 1;
    const size_t nodes = (size_t)(cfg->max_nodes > 0 ? cfg->max_nodes : 1);
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#else
    (void)threads;
#endif
    uint32_t *bitmap_a = malloc((size_t)C * node_chunks * 4), *bitmap_b = malloc((size_t)C * node_chunks * 4);
    uint8_t *x_int = layers > 0 ? malloc(nodes * 2 * (size_t)cfg->message_size) : NULL;
    uint32_t *packed = layers > 0 ? malloc((size_t)layers * nodes * message_chunks * 4) : NULL; /* kept per layer for K10 */
    int32_t *n_incl = malloc((size_t)C * 4), *clause_node = malloc((size_t)C * 4), *updates = malloc((size_t)K * C * 4);
    int32_t *sums = malloc((size_t)K * 4);
    int rc = 0;
    if (!bitmap_a || !bitmap_b || !n_incl || !clause_node || !updates || !sums || (layers > 0 && (!x_int || !packed))) rc = -1;
    for (int32_t i = 0; rc == 0 && i < n; ++i) {
        const int32_t e = graph_ids[i];
        const uint32_t step = (uint32_t)(first_step + (uint64_t)i);
        const int n_nodes = (int)g->number_of_graph_nodes[e];
        const size_t base = g->node_index[e];
        const uint32_t *types = g->node_type + base;
        /* evaluation, keeping every layer's messages (tm.py:563-662) */
        uint32_t *now = bitmap_a, *next = bitmap_b;
        clause_node_bits(C, node_chunks, la_chunks, cfg->state_bits, filter, ta_state, types, g->number_of_node_types,
                         n_nodes, g->X + base * la_chunks, NULL, now);
        for (int c = 0; c < C; ++c) n_incl[c] = include_count(ta_state, c, la_chunks, cfg->state_bits, filter);
        for (int layer = 0; layer < layers; ++layer) {
            uint32_t *messages = packed + (size_t)layer * nodes * message_chunks;
            const uint32_t *n_edges = g->number_of_graph_node_edges + base;
            const uint32_t *edges = n_nodes > 0 ? g->edge + (size_t)g->edge_index[base] * 2 : g->edge;
            build_messages(cfg, node_chunks, n_nodes, hypervectors, now, n_edges, edges, x_int, messages);
            clause_node_bits(C, node_chunks, message_chunks, cfg->state_bits, message_filter, message_ta_state[layer],
                             types, g->number_of_node_types, n_nodes, messages, now, next);
            for (int c = 0; c < C; ++c)
                n_incl[c] += include_count(message_ta_state[layer], c, message_chunks, cfg->state_bits, message_filter);
            uint32_t *swap = now;
            now = next;
            next = swap;
        }
        class_sums(cfg, node_chunks, n_nodes, now, clause_weights, sums);
        /* K7: a uniformly drawn true node per clause, -1 without one.  Draw: word 0 at counter
         * (clause, 0, step, TAG_CLAUSE_NODE); index = (draw * count) >> 32 among the true nodes. */
#pragma omp parallel for schedule(static)
        for (int c = 0; c < C; ++c) {
            int count = 0;
            for (int node = 0; node < n_nodes; ++node) count += (now[(size_t)c * node_chunks + node / 32] >> (node % 32)) & 1u;
            clause_node[c] = -1;
            if (count > 0) {
                uint32_t r[4];
                philox4x32_10((uint32_t)c, 0u, step, TAG_CLAUSE_NODE, k0, k1, r);
                int pick = (int)(((uint64_t)r[0] * (uint64_t)count) >> 32);
                for (int node = 0; node < n_nodes; ++node)
                    if ((now[(size_t)c * node_chunks + node / 32] >> (node % 32)) & 1u) {
                        if (pick == 0) {
                            clause_node[c] = node;
                            break;
                        }
                        --pick;
                    }
            }
        }
        /* K8.  Draws at counter (clause, class, step, TAG_CLAUSE_UPDATES): word 0 gates negative
         * targets, word 1 gates on the error, kept when draw * 2T < |y - sum| * 2^32. */
        const int32_t *y = encoded_Y + (size_t)e * K;
        for (int k = 0; k < K; ++k) {
            const int64_t cs = sums[k] > T ? T : sums[k] < -T ? -T : sums[k];
            const int target = 1 - 2 * (cs > y[k]);
            const int64_t err = y[k] > cs ? y[k] - cs : cs - y[k];
            for (int c = 0; c < C; ++c) {
                int32_t *w = clause_weights + (size_t)k * C + c;
                const int sign = *w >= 0 ? 1 : -1;
                uint32_t r[4];
                philox4x32_10((uint32_t)c, (uint32_t)k, step, TAG_CLAUSE_UPDATES, k0, k1, r);
                const int skip = (target == -1 && (uint64_t)r[0] >= t->q_threshold) ||
                                 ((uint64_t)r[1] * (uint64_t)(2 * (int64_t)T) >= ((uint64_t)err << 32));
                const int u = skip ? 0 : target * sign;
                const int fired = clause_node[c] != -1;
                if (u > 0 && fired && (*w < 0 ? -(int64_t)*w : (int64_t)*w) < 2147483647) {
                    *w += sign;
                } else if (u < 0 && fired) {
                    int64_t moved = (int64_t)*w - sign;
                    if (t->negative_clauses == 0 && moved < 1) moved = 1;
                    *w = (int32_t)moved;
                }
                updates[(size_t)k * C + c] = u;
            }
        }
        /* K9, K10 */
        feedback(cfg, t, step, 0, ta_state, la_chunks, clause_node, n_incl, g->X + base * la_chunks, updates);
        for (int layer = 0; layer < layers; ++layer)
            feedback(cfg, t, step, layer + 1, message_ta_state[layer], message_chunks, clause_node, n_incl,
                     packed + (size_t)layer * nodes * message_chunks, updates);
    }
    free(bitmap_a);
    free(bitmap_b);
    free(x_int);
    free(packed);
    free(n_incl);
    free(clause_node);
    free(updates);
    free(sums);
    return rc;
}

/* Threads a call may use: the processors OpenMP sees, capped by OMP_NUM_THREADS.  (Not
 * omp_get_max_threads(): the entry points above set the calling thread's team size, and that
 * setting outlives the call.) */
int gtmc_threads_available(void) {
#ifdef _OPENMP
    int n = omp_get_num_procs();
    const char *env = getenv("OMP_NUM_THREADS");
    if (env) {
        const int k = atoi(env);
        if (k > 0 && k < n) n = k;
    }
    return n > 0 ? n : 1;
#else
    return 1;
#endif
}
