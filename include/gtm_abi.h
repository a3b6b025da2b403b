/*
 * C ABI of the MI355X Graph Tsetlin Machine hot path (libgtm_hip.so).
 *
 * The reference has no C interface: its operator boundary is PyCUDA's
 * `fn.prepared_call(grid, block, *args)` on kernels JIT-compiled from
 * GraphTsetlinMachine/kernels.py with the model's hyper-parameters baked in as
 * #defines (tm.py:437-513).  Each entry point below replaces one of those
 * prepared kernels (or one of the driver loops that chain them) and cites it.
 * The #defines travel in `gtm_config`; grid/block shapes are chosen inside.
 *
 * Conventions
 *  - every pointer inside the structs and in the argument lists is a DEVICE
 *    pointer owned by the caller (the Python side takes them from torch
 *    tensors); the library never allocates or frees device memory;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *    all work is enqueued on it.  Only gtm_fit and the two single-graph
 *    training operators that take an example index wait for the stream (to
 *    read the example's size, and gtm_fit also to report a failed run);
 *  - the return value is GTM_OK or an error code; gtm_last_error() gives the
 *    text for the calling thread.  No C++ exception crosses the boundary;
 *  - memory layouts are the reference's: X uint32 [nodes][LA_CHUNKS];
 *    ta_state uint32 [CLAUSES][chunks][STATE_BITS] (bit-sliced, top plane =
 *    include mask); clause_weights int32 [CLASSES][CLAUSES]; clause/node
 *    bitmaps uint32 [CLAUSES][NODE_CHUNKS] per graph; packed messages uint32
 *    [max_nodes][MESSAGE_CHUNKS] per graph;
 *  - random decisions come from Philox4x32-10 keyed by `seed` and addressed by
 *    (clause, class or word, training step, purpose); they do not depend on
 *    the launch shape.
 */
#ifndef GTM_ABI_H
#define GTM_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GTM_ABI_VERSION 3
#define GTM_MAX_DEPTH 8

#define GTM_OK 0
#define GTM_ERR_INVALID 1 /* bad argument or configuration */
#define GTM_ERR_HIP 2     /* a HIP call or kernel launch failed */

/* The macros injected at tm.py:438-464, plus depth, s and the RNG seed. */
typedef struct gtm_config {
    int32_t classes;                      /* CLASSES */
    int32_t clauses;                      /* CLAUSES */
    int32_t literals;                     /* LITERALS = 2 * hypervector_size */
    int32_t state_bits;                   /* STATE_BITS (1..32) */
    int32_t boost_true_positive_feedback; /* BOOST_TRUE_POSITIVE_FEEDBACK */
    int32_t threshold;                    /* THRESHOLD (T) */
    int32_t max_included_literals;        /* MAX_INCLUDED_LITERALS */
    int32_t negative_clauses;             /* NEGATIVE_CLAUSES */
    int32_t max_nodes;                    /* MAX_NODES: bitmap row stride = ceil(max_nodes/32) words */
    int32_t message_size;                 /* MESSAGE_SIZE */
    int32_t message_bits;                 /* MESSAGE_BITS */
    int32_t depth;                        /* number of layers (tm.py:62) */
    double q;                             /* Q */
    double s[GTM_MAX_DEPTH];              /* s per layer (tm.py:63-66) */
    uint64_t seed;                        /* Philox key */
} gtm_config;

/* gtm_graphs.flags: on every node, literal k + LITERALS/2 is the complement of
 * literal k (what Graphs builds, graphs.py:91-98,148-159: a property sets k and
 * clears its negation), and every graph has at least one node.  With it the
 * tile kernels may keep only the positive literals' rows on chip.  Check with
 * gtm_graphs_properties(); never set it for data the check has not passed. */
#define GTM_GRAPHS_COMPLEMENTARY 1

/* Device copies of the arrays of a Graphs object (graphs.py:38,101-112,128-129). */
typedef struct gtm_graphs {
    const uint32_t *X;                          /* [total_nodes][LA_CHUNKS] */
    const uint32_t *node_type;                  /* [total_nodes] */
    const uint32_t *number_of_graph_node_edges; /* [total_nodes] */
    const uint32_t *edge;                       /* [total_edges][2] = (destination, type) */
    const uint32_t *node_index;                 /* [number_of_graphs] */
    const uint32_t *edge_index;                 /* [total_nodes] */
    const uint32_t *number_of_graph_nodes;      /* [number_of_graphs] */
    int32_t number_of_graphs;
    int32_t number_of_node_types;      /* Graphs.number_of_node_types() */
    int32_t max_number_of_graph_nodes; /* must be <= gtm_config.max_nodes */
    int32_t flags;                     /* GTM_GRAPHS_* bits the caller vouches for; 0 is always valid */
    int64_t total_nodes;
    int64_t total_edges;
    const uint32_t *tiles; /* optional: literal-major tiles from gtm_build_tiles, or NULL */
} gtm_graphs;

/* The model's device buffers (tm.py:110-124). */
typedef struct gtm_state {
    uint32_t *ta_state;                            /* [CLAUSES][LA_CHUNKS][STATE_BITS] */
    uint32_t *message_ta_state[GTM_MAX_DEPTH - 1]; /* [CLAUSES][MESSAGE_CHUNKS][STATE_BITS] each */
    int32_t *clause_weights;                       /* [CLASSES][CLAUSES] */
    const uint32_t *hypervectors;                  /* [CLAUSES][MESSAGE_BITS] */
} gtm_state;

int gtm_abi_version(void);
const char *gtm_last_error(void);

/* ---- one entry point per reference kernel ------------------------------ */

/* `prepare` (kernels.py:638-664; called at tm.py:518,525): TA bank to state
 * 2^(B-1)-1, weights to random +-1 (NEGATIVE_CLAUSES == 1) or 1. */
int gtm_prepare(const gtm_config *cfg, uint64_t step, uint32_t *ta_state, int32_t *clause_weights, void *stream);

/* `prepare_message_ta_state` (kernels.py:622-636; tm.py:521). */
int gtm_prepare_message_ta_state(const gtm_config *cfg, uint32_t *message_ta_state, void *stream);

/* `calculate_messages` (kernels.py:407-468; tm.py:582-593) for graphs
 * [first_graph, first_graph + n_graphs): clause_node_output is
 * [n_graphs][CLAUSES][NODE_CHUNKS]; number_of_include_actions [CLAUSES] may
 * be NULL.  include_plane is caller-provided scratch of LA_CHUNKS * CLAUSES
 * words; it receives the bank's include masks word-major ([chunk][clause]),
 * the form the evaluation kernel reads coalesced. */
int gtm_calculate_messages(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph, int32_t n_graphs,
                           const uint32_t *ta_state, uint32_t *include_plane, uint32_t *clause_node_output,
                           int32_t *number_of_include_actions, void *stream);

/* `prepare_messages` + `exchange_messages` + `encode_messages`
 * (kernels.py:532-615; tm.py:599-630) fused: writes the packed message
 * literals clause_X [n_graphs][max_nodes][MESSAGE_CHUNKS] directly, without
 * the one-int-per-literal scratch. */
int gtm_exchange_messages(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph, int32_t n_graphs,
                          const uint32_t *hypervectors, const uint32_t *clause_node_output, uint32_t *clause_X,
                          void *stream);

/* `calculate_messages_conditional` (kernels.py:470-530; tm.py:633-645).
 * number_of_include_actions (may be NULL) is incremented; include_plane is
 * scratch of MESSAGE_CHUNKS * CLAUSES words as above. */
int gtm_calculate_messages_conditional(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph,
                                       int32_t n_graphs, const uint32_t *message_ta_state, uint32_t *include_plane,
                                       const uint32_t *clause_node_output_condition, uint32_t *clause_node_output,
                                       int32_t *number_of_include_actions, const uint32_t *clause_X, void *stream);

/* `evaluate` (kernels.py:279-317; tm.py:652-659) including the zeroing of
 * class_sum that the driver does from the host (tm.py:578-579): class_sum is
 * [n_graphs][CLASSES], overwritten. */
int gtm_evaluate(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph, int32_t n_graphs,
                 const uint32_t *clause_node_output, const int32_t *clause_weights, int32_t *class_sum,
                 void *stream);

/* `select_clause_node` (kernels.py:319-354; tm.py:693-700) for graph `example`. */
int gtm_select_clause_node(const gtm_config *cfg, const gtm_graphs *graphs, int32_t example, uint64_t step,
                           const uint32_t *clause_node_output, int32_t *clause_node, void *stream);

/* `select_clause_updates` (kernels.py:356-405; tm.py:704-714). encoded_Y is
 * [number_of_graphs][CLASSES]; class_clause_update [CLASSES][CLAUSES]. */
int gtm_select_clause_updates(const gtm_config *cfg, uint64_t step, int32_t *clause_weights,
                              const int32_t *class_sum, const int32_t *encoded_Y, int32_t example,
                              const int32_t *clause_node, int32_t *class_clause_update, void *stream);

/* `update` (kernels.py:213-242; tm.py:718-730): Type I/II feedback on the
 * layer-0 bank with s = cfg->s[0]. */
int gtm_update(const gtm_config *cfg, const gtm_graphs *graphs, int32_t example, uint64_t step,
               uint32_t *ta_state, const int32_t *clause_node, const int32_t *number_of_include_actions,
               const int32_t *class_clause_update, void *stream);

/* `update_message` (kernels.py:185-211; tm.py:735-746) on message bank
 * `bank` (1 .. depth-1) with s = cfg->s[bank]; clause_X is that layer's
 * [max_nodes][MESSAGE_CHUNKS] block for the example. */
int gtm_update_message(const gtm_config *cfg, uint64_t step, int32_t bank, uint32_t *message_ta_state,
                       const int32_t *clause_node, const int32_t *number_of_include_actions,
                       const uint32_t *clause_X, const int32_t *class_clause_update, void *stream);

/* ---- the driver loops --------------------------------------------------- */

/* A second, derived layout of a data set for batched depth-1 inference: per
 * tile of graphs one bit-row per literal over the tile's node slots (plus one
 * row per node type), so that a clause is evaluated as the AND of the rows of
 * its included literals only.  Stands where the reference uploads X once per
 * data set (tm.py:759-763).  gtm_tiles_bytes() is 0 when the data set's shape
 * has no such layout (then leave gtm_graphs.tiles NULL); gtm_build_tiles()
 * fills a caller-owned buffer of that size from X / node_type. */
size_t gtm_tiles_bytes(const gtm_config *cfg, const gtm_graphs *graphs);

/* No counterpart in the reference (its kernels read X as it is).  Looks at the
 * data set once on the device: properties[0] = 1 if on some node a negated
 * literal is not the complement of its positive one, properties[1] = 1 if
 * some graph has no nodes (two uint32 in device memory).  Both 0 entitles the
 * caller to set GTM_GRAPHS_COMPLEMENTARY before gtm_tiles_bytes /
 * gtm_build_tiles and in every later call with that data set. */
int gtm_graphs_properties(const gtm_config *cfg, const gtm_graphs *graphs, uint32_t *properties, void *stream);
int gtm_build_tiles(const gtm_config *cfg, const gtm_graphs *graphs, uint32_t *tiles, void *stream);

/* Scratch needed by gtm_score for sub-batches of `batch` graphs. */
size_t gtm_score_workspace_bytes(const gtm_config *cfg, const gtm_graphs *graphs, int32_t batch);

/* `_score` (tm.py:786-812): class sums [n_graphs][CLASSES] of graphs
 * [first_graph, first_graph + n_graphs), evaluated `batch` graphs at a time.
 * With depth == 1 and graphs->tiles set, one fused kernel evaluates all
 * clauses and accumulates the class sums without writing a bitmap. */
int gtm_score(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, int32_t first_graph,
              int32_t n_graphs, int32_t batch, void *workspace, size_t workspace_bytes, int32_t *class_sum,
              void *stream);

/* No counterpart in the reference.  gtm_score for callers that cannot allocate
 * device memory or hand over a workspace of their own: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same
 * arguments and results as gtm_score, minus the workspace: the scratch is a
 * fixed array inside the library's device image (gtm_score_static_scratch_bytes()
 * = 16 MiB on every GPU the library runs on, held until the process ends).  A
 * model and batch whose gtm_score_workspace_bytes() exceeds that is refused
 * with GTM_ERR_INVALID.  The call allocates and frees nothing.  All calls on
 * one GPU share the array: calls that overlap on one GPU (other streams, other
 * threads) race; calls one after the other need nothing cleared between them. */
size_t gtm_score_static_scratch_bytes(void);
int gtm_score_static(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, int32_t first_graph,
                     int32_t n_graphs, int32_t batch, int32_t *class_sum, void *stream);

/* Scratch needed by gtm_fit. */
size_t gtm_fit_workspace_bytes(const gtm_config *cfg, const gtm_graphs *graphs);

/* The inner loop of `_fit` (tm.py:669-747) over examples
 * [first_example, first_example + n_examples), strictly in order (online
 * learning: example e+1 sees the state left by e).  Example i uses training
 * step first_step + i for its random draws.  With depth == 1 and
 * graphs->tiles set the whole run is one cooperative launch in which each
 * workgroup keeps its clauses' automata in LDS and the class sums are the
 * only exchange between workgroups.  Models with message layers whose
 * MESSAGE_SIZE is a multiple of 32 run the same way, with one more exchange
 * per layer; when a workgroup owns several clauses the run is a few such
 * launches, of 256 to 2,048 examples, and the clauses are shared out among the
 * workgroups anew before each.  The waits are bounded (5 s of the device's
 * wall clock): if one runs out, the model is put back as it was before that
 * launch and the remaining examples are trained by launches per example
 * instead, which wait for nobody - same results, the call still returns
 * GTM_OK. */
int gtm_fit(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, const int32_t *encoded_Y,
            int32_t first_example, int32_t n_examples, uint64_t first_step, void *workspace,
            size_t workspace_bytes, void *stream);

/* ---- measurement -------------------------------------------------------- */

/* `get_ta_states` and `get_hyperliterals` (kernels.py:718-757, :761-790; called
 * from tm.py:144-205): the integer state (resp. 1 for an include action) of
 * every automaton of a bank, uint32 out[CLAUSES][literals].  `chunks` and
 * `literals` are the bank's: LA_CHUNKS / LITERALS for ta_state, MESSAGE_CHUNKS /
 * MESSAGE_LITERALS for a message bank. */
int gtm_get_ta_states(const gtm_config *cfg, const uint32_t *bank, int32_t chunks, int32_t literals, uint32_t *out,
                      void *stream);
int gtm_get_hyperliterals(const gtm_config *cfg, const uint32_t *bank, int32_t chunks, int32_t literals,
                          uint32_t *out, void *stream);

/* The loops of `transform` and `transform_nodewise` (tm.py:814-900 with
 * kernels.py:671-710) for graphs [first_graph, first_graph + n_graphs), `batch`
 * graphs per launch: int32 transformed[n_graphs][CLAUSES] = 1 where the clause
 * is true at some node of the graph; when `nodewise` is not NULL also int32
 * nodewise[n_graphs][CLAUSES][width] = the clause's truth at every node (0 past
 * the graph's nodes; width >= the largest graph of the range); and the class
 * sums as gtm_score gives them.  Workspace: gtm_transform_workspace_bytes(). */
size_t gtm_transform_workspace_bytes(const gtm_config *cfg, const gtm_graphs *graphs, int32_t batch);
int gtm_transform(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, int32_t first_graph,
                  int32_t n_graphs, int32_t batch, void *workspace, size_t workspace_bytes, int32_t *transformed,
                  int32_t *nodewise, int32_t width, int32_t *class_sum, void *stream);

/* No counterpart in the reference (its tuning knobs are the `grid` and `block` constructor
 * arguments, tm.py:53-54).  The library's tuning and test switches - the GTM_* names listed in its
 * documentation - are read from the process environment once, when the library is loaded, and
 * never again by the entry points above.  gtm_tuning_set() sets one switch for the rest of the
 * process (value NULL = not set), gtm_tuning_get() returns its value or NULL, gtm_tuning_reload()
 * reads the environment again.  For tests and tuning runs: none of the three may run while another
 * call of the library is under way. */
int gtm_tuning_set(const char *name, const char *value);
const char *gtm_tuning_get(const char *name);
int gtm_tuning_reload(void);

/* No counterpart in the reference.  While enabled, gtm_score / gtm_transform /
 * gtm_fit bracket the launches of the kernels that do their work (clause
 * evaluation per layer, message construction, the one-launch training kernels)
 * with HIP events on the caller's stream, each under its kernel's name (at most
 * 4096 launches are kept; gtm_score_static never records any).  gtm_profile_read() waits for those events, returns
 * the name of the kernel launched last, the number of launches seen and their
 * summed duration (all kernels together: a model without message layers has one),
 * and clears the record.  Not thread-safe; meant for the benchmark. */
int gtm_profile_enable(int on);
int gtm_profile_read(const char **kernel_name, int32_t *launches, double *total_ms);
/* The same measurement kernel by kernel, without ending it: the index-th distinct kernel name in
 * the order of first launch, the number of its launches and their total duration.  An index past
 * the last name gives *kernel_name = NULL and zeros.  (No counterpart in the reference.) */
int gtm_profile_read_kernel(int32_t index, const char **kernel_name, int32_t *launches, double *total_ms);

#ifdef __cplusplus
}
#endif
#endif /* GTM_ABI_H */
