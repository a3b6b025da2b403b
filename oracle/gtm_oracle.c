/* CPU restatement in plain C of the Graph Tsetlin Machine's inference path.
 *
 * TEST INFRASTRUCTURE ONLY: nothing in the shipped package links or loads this
 * file.  It is a second, independent checker next to oracle/gtm_oracle.py (the
 * two are compared with each other in tests/test_oracle_c.py) and the CPU
 * baseline that bench.py times beside the GPU.
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

int gtmc_threads_available(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
