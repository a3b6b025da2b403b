// Graph Tsetlin Machine hot path for gfx950 (MI355X): HIP kernels and the
// C ABI declared in include/gtm_abi.h.
//
// All arithmetic is 32-bit bitwise/integer work on wave64; nothing here is
// GEMM-shaped, so no MFMA.  Layouts are the reference's (see gtm_abi.h).
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <mutex>
#include <string>
#include <unordered_map>

#include "../../include/gtm_abi.h"
#include "philox.h"
#include "score_tiles.h"
#include "score_narrow.h"
#include "score_messages.h"

namespace {

// ------------------------------------------------------------------ errors

// Plain storage: nothing of this library's has a destructor that runs at thread or process exit.
thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

// Set by blocks_for() when a work size does not fit the grid of one launch; the launch that follows
// runs one block (harmless) and check_launch() reports the call as failed.
thread_local bool g_grid_overflow = false;

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (g_grid_overflow) {
        g_grid_overflow = false;
        return fail(GTM_ERR_INVALID, "%s: the work size exceeds what one launch can cover (2^31 - 1 blocks); "
                                     "pass fewer graphs per call", what);
    }
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return GTM_OK;
}

// ------------------------------------------------------------------ switches
// Tuning and test aids.  The process environment is read ONCE, when the library is loaded; the
// entry points then only look at this table.  gtm_tuning_set / gtm_tuning_reload (tests, tuning
// runs) change it, and must not run while another call of the library is under way.
#define GTM_SWITCHES(X) \
    X(FIT_DEEP_CHUNK) \
    X(FIT_DEEP_CLAUSES_PER_GROUP) \
    X(FIT_DEEP_IN_MEMORY) \
    X(FIT_DEEP_NO_DEAL) \
    X(FIT_DEEP_NO_MASKS) \
    X(FIT_DEEP_WINDOW_ROWS) \
    X(FIT_FACTOR_MIN) \
    X(FIT_PER_GROUP) \
    X(FIT_SPIN_LIMIT) \
    X(HALF_LANE_WORDS) \
    X(MESSAGES_IN_LDS) \
    X(NARROW_IN_ORDER) \
    X(NARROW_READS) \
    X(NARROW_ROWS_AS_STORED) \
    X(NODE_MESSAGES_BY_ATOMICS) \
    X(NO_DEEP_FIT) \
    X(NO_DEEP_PERSISTENT_FIT) \
    X(NO_DIRECT_FIT) \
    X(NO_FUSED_MESSAGES) \
    X(NO_HALF_ROWS) \
    X(NO_HALF_TILES) \
    X(NO_LISTS_IN_LDS) \
    X(NO_NARROW_TWO_PHASE) \
    X(NO_NARROW_LAYERS) \
    X(NO_PERSISTENT_FIT) \
    X(NO_SMALL_FIT) \
    X(NO_TILE_LINE) \
    X(TILE_LINE_GROUPS) \
    X(NO_TILE_PACK) \
    X(NO_TILE_TRANSFORM) \
    X(NO_TWO_PHASE) \
    X(TILE_LANE_WORDS) \
    X(WIDE_SPLITS) \
    X(WIDE_WALK_FACTOR)

enum Switch {
#define X(name) T_##name,
    GTM_SWITCHES(X)
#undef X
    T_COUNT
};
const char *const g_switch_name[T_COUNT] = {
#define X(name) "GTM_" #name,
    GTM_SWITCHES(X)
#undef X
};
struct Switches {
    bool set[T_COUNT];
    char value[T_COUNT][24];
    void put(int i, const char *v) {
        set[i] = v != nullptr;
        snprintf(value[i], sizeof value[i], "%s", v ? v : "");
    }
    Switches() {
        for (int i = 0; i < T_COUNT; ++i) put(i, getenv(g_switch_name[i]));
    }
};
Switches g_switches;  // filled from the environment when the library is loaded

// The switch's value, or NULL when it is not set (what getenv gave when this was read per call).
inline const char *tune(Switch which) { return g_switches.set[which] ? g_switches.value[which] : nullptr; }

// --------------------------------------------------------------- profiling
// When enabled (gtm_profile_enable), the launches of the kernels that do the work of a
// driver loop are bracketed by HIP events on the caller's stream, each under its kernel's name.

struct Profile {
    bool on = false;
    const char *name = "";
    static constexpr int MAX = 4096;
    hipEvent_t start[MAX], stop[MAX];
    const char *name_of[MAX];
    int created = 0, used = 0;
};
Profile g_prof;

// Set for the duration of a call that must create no events (gtm_score_static): per thread, so that
// other threads' calls and the global switch are left alone.
thread_local bool g_prof_quiet = false;

void profile_start(const char *name, hipStream_t st) {
    if (!g_prof.on || g_prof_quiet || g_prof.used >= Profile::MAX) return;
    if (g_prof.used >= g_prof.created) {
        if (hipEventCreate(&g_prof.start[g_prof.created]) != hipSuccess) return;
        if (hipEventCreate(&g_prof.stop[g_prof.created]) != hipSuccess) {
            (void)hipEventDestroy(g_prof.start[g_prof.created]);
            return;
        }
        ++g_prof.created;
    }
    g_prof.name = name;
    g_prof.name_of[g_prof.used] = name;
    (void)hipEventRecord(g_prof.start[g_prof.used], st);
}

void profile_stop(hipStream_t st) {
    if (!g_prof.on || g_prof_quiet || g_prof.used >= g_prof.created) return;
    (void)hipEventRecord(g_prof.stop[g_prof.used], st);
    ++g_prof.used;
}

// --------------------------------------------------------- derived constants

struct Dims {
    int K, C, LA, MC, NC, B, MB, M;
    uint32_t filter, mfilter;
};

uint32_t tail_filter(int bits) {
    int r = bits % 32;
    return r == 0 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << r);
}

int validate(const gtm_config *cfg, Dims *d) {
    if (!cfg) return fail(GTM_ERR_INVALID, "cfg is NULL");
    if (cfg->classes < 1 || cfg->classes > 65535) return fail(GTM_ERR_INVALID, "classes=%d out of range", cfg->classes);
    if (cfg->clauses < 1) return fail(GTM_ERR_INVALID, "clauses=%d", cfg->clauses);
    if (cfg->literals < 1) return fail(GTM_ERR_INVALID, "literals=%d", cfg->literals);
    if (cfg->state_bits < 1 || cfg->state_bits > 32) return fail(GTM_ERR_INVALID, "state_bits=%d out of 1..32", cfg->state_bits);
    if (cfg->threshold < 1) return fail(GTM_ERR_INVALID, "threshold=%d", cfg->threshold);
    if (cfg->max_nodes < 1) return fail(GTM_ERR_INVALID, "max_nodes=%d", cfg->max_nodes);
    if (cfg->depth < 1 || cfg->depth > GTM_MAX_DEPTH) return fail(GTM_ERR_INVALID, "depth=%d out of 1..%d", cfg->depth, GTM_MAX_DEPTH);
    if (cfg->message_size < 1 || cfg->message_bits < 1) return fail(GTM_ERR_INVALID, "message_size/message_bits must be >= 1");
    if (cfg->message_bits > 64) return fail(GTM_ERR_INVALID, "message_bits=%d > 64", cfg->message_bits);
    d->K = cfg->classes;
    d->C = cfg->clauses;
    d->LA = (cfg->literals - 1) / 32 + 1;
    d->MC = (2 * cfg->message_size - 1) / 32 + 1;
    d->NC = (cfg->max_nodes - 1) / 32 + 1;
    d->B = cfg->state_bits;
    d->MB = cfg->message_bits;
    d->M = cfg->message_size;
    d->filter = tail_filter(cfg->literals);
    d->mfilter = tail_filter(2 * cfg->message_size);
    return GTM_OK;
}

int validate_graphs(const gtm_config *cfg, const gtm_graphs *g, int first, int n) {
    if (!g) return fail(GTM_ERR_INVALID, "graphs is NULL");
    if (!g->X || !g->node_type || !g->node_index || !g->number_of_graph_nodes)
        return fail(GTM_ERR_INVALID, "graphs has NULL arrays");
    if (g->number_of_node_types < 1) return fail(GTM_ERR_INVALID, "number_of_node_types=%d", g->number_of_node_types);
    if (g->max_number_of_graph_nodes > cfg->max_nodes)
        return fail(GTM_ERR_INVALID, "graphs hold up to %d nodes but the model was sized for max_nodes=%d",
                    g->max_number_of_graph_nodes, cfg->max_nodes);
    if (first < 0 || n < 0 || (int64_t)first + n > g->number_of_graphs)
        return fail(GTM_ERR_INVALID, "graph range [%d, %d) outside 0..%d", first, first + n, g->number_of_graphs);
    return GTM_OK;
}

uint32_t feedback_threshold(double s) {
    double t = 65536.0 / s;
    if (!(t < 65536.0)) return 65536u;
    if (t < 0.0) return 0u;
    return (uint32_t)t;
}

uint64_t q_threshold(double q, int classes) {
    double p = q / (double)(classes - 1 > 1 ? classes - 1 : 1);
    if (p > 1.0) p = 1.0;
    if (p < 0.0) p = 0.0;
    return (uint64_t)(p * 4294967296.0);
}

inline unsigned blocks_for(int64_t items, int per_block) {
    const int64_t blocks = (items + per_block - 1) / per_block;
    if (blocks > 0x7FFFFFFF) {  // never truncated silently
        g_grid_overflow = true;
        return 1u;
    }
    return (unsigned)blocks;
}

constexpr int TPB = 256;

__device__ __forceinline__ int chunks_of(int n) { return n == 0 ? 1 : (n - 1) / 32 + 1; }  // C division of kernels.py:289
__device__ __forceinline__ uint32_t node_filter_of(int n) {
    int r = n % 32;
    return r == 0 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << r);
}

// ------------------------------------------------------------------ kernels

// K11/K12: every automaton to state 2^(B-1)-1; optional weights.
__global__ void k_prepare_bank(uint32_t *bank, int64_t words, int B) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < words) bank[i] = ((int)(i % B) == B - 1) ? 0u : 0xFFFFFFFFu;
}

__global__ void k_prepare_weights(int32_t *w, int K, int C, int negative, uint32_t k0, uint32_t k1, uint32_t step) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= K * C) return;
    int class_id = i / C, clause = i % C;
    int v = 1;
    if (negative == 1) {
        philox_out r = philox4x32_10((uint32_t)clause, (uint32_t)class_id, step, GTM_TAG_PREPARE, k0, k1);
        v = 1 - 2 * (int)(r.v[0] & 1u);
    }
    w[i] = v;
}

// Include plane of a bank, word-major ([chunk][clause]) so that lanes that
// hold consecutive clauses read consecutive addresses; also the include count
// of kernels.py:251-277.
__global__ void k_include_plane(const uint32_t *__restrict__ bank, int C, int chunks, int B, uint32_t filter,
                                uint32_t *__restrict__ inc_t, int32_t *n_incl, int accumulate) {
    int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    int count = 0;
    for (int w = 0; w < chunks; ++w) {
        uint32_t v = bank[((int64_t)c * chunks + w) * B + (B - 1)];
        if (w == chunks - 1) v &= filter;
        inc_t[(int64_t)w * C + c] = v;
        count += __popc(v);
    }
    if (n_incl) n_incl[c] = accumulate ? n_incl[c] + count : count;
}

// K1 / K2: truth of clause c at the <=32 nodes of chunk nc of graph b.
// rows_mode 0: literal rows are X rows of the graph (base node_index[g]);
// rows_mode 1: literal rows are the graph's packed messages (base b*max_nodes).
template <int REG_CHUNKS>
__global__ void k_clause_node_bits(const uint32_t *__restrict__ inc_t, int C, int chunks, const uint32_t *__restrict__ rows,
                                   int rows_mode, int max_nodes, const uint32_t *__restrict__ node_type, int n_types,
                                   const uint32_t *__restrict__ node_index, const uint32_t *__restrict__ n_nodes_arr,
                                   int first_graph, int NC, const uint32_t *__restrict__ cond, uint32_t *__restrict__ out,
                                   int clause_blocks) {
    int64_t blk = blockIdx.x;
    int cb = (int)(blk % clause_blocks);
    int64_t rest = blk / clause_blocks;
    int nc = (int)(rest % NC);
    int b = (int)(rest / NC);
    int c = cb * blockDim.x + threadIdx.x;
    if (c >= C) return;
    int g = first_graph + b;
    int n = (int)n_nodes_arr[g];
    int64_t base = (int64_t)node_index[g];
    const uint32_t *rbase = rows_mode == 0 ? rows + base * chunks : rows + (int64_t)b * max_nodes * chunks;
    uint32_t word;
    if (nc >= chunks_of(n) || n == 0) {
        word = 0xFFFFFFFFu;  // kernels.py:443-466: chunks past the graph are left all ones
    } else {
        uint32_t inc[REG_CHUNKS > 0 ? REG_CHUNKS : 1];
        if (REG_CHUNKS > 0) {
#pragma unroll
            for (int w = 0; w < REG_CHUNKS; ++w) inc[w] = w < chunks ? inc_t[(int64_t)w * C + c] : 0u;
        }
        int my_type = c % n_types;
        word = 0;
        int node0 = nc * 32;
        int lim = n - node0 < 32 ? n - node0 : 32;
        for (int p = 0; p < lim; ++p) {
            int node = node0 + p;
            const uint32_t *row = rbase + (int64_t)node * chunks;  // uniform across the wave
            uint32_t violated = 0;
            if (REG_CHUNKS > 0) {
#pragma unroll
                for (int w = 0; w < REG_CHUNKS; ++w)
                    if (w < chunks) violated |= inc[w] & ~row[w];
            } else {
                for (int w = 0; w < chunks; ++w) violated |= inc_t[(int64_t)w * C + c] & ~row[w];
            }
            bool ok = violated == 0 && (int)node_type[base + node] == my_type;
            word |= (uint32_t)ok << p;
        }
    }
    int64_t o = ((int64_t)b * C + c) * NC + nc;
    if (cond) word &= cond[o];
    out[o] = word;
}

// K3: packed messages start as "no message": positive half 0, negated half 1.
__global__ void k_messages_blank(uint32_t *clause_X, int64_t words, int MC, int M) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= words) return;
    int m = (int)(i % MC);
    int lo = m * 32, hi = lo + 32;
    int a = lo > M ? lo : M, z = hi < 2 * M ? hi : 2 * M;
    uint32_t v = 0;
    if (a < z) {
        int len = z - a;
        uint32_t ones = len == 32 ? 0xFFFFFFFFu : ((1u << len) - 1u);
        v = ones << (a - lo);
    }
    clause_X[i] = v;
}

// K4 (+K5): each true (clause, source node) sets, at every out-neighbour, the
// clause's hypervector bits rotated by the edge type and clears their
// negations (kernels.py:571-588), straight into the packed words.
__global__ void k_messages_scatter(const uint32_t *__restrict__ bitmap, int C, int NC, const uint32_t *__restrict__ hv,
                                   int MB, int M, int MC, int max_nodes, const uint32_t *__restrict__ node_index,
                                   const uint32_t *__restrict__ n_nodes_arr, const uint32_t *__restrict__ n_edges,
                                   const uint32_t *__restrict__ edge_index, const uint32_t *__restrict__ edge,
                                   int first_graph, int64_t total, uint32_t *clause_X) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int nc = (int)(i % NC);
    int64_t rest = i / NC;
    int c = (int)(rest % C);
    int b = (int)(rest / C);
    int g = first_graph + b;
    int n = (int)n_nodes_arr[g];
    if (n == 0 || nc >= chunks_of(n)) return;
    uint32_t word = bitmap[i];
    if (nc == chunks_of(n) - 1) word &= node_filter_of(n);
    if (word == 0) return;
    int64_t base = (int64_t)node_index[g];
    uint32_t *cx = clause_X + (int64_t)b * max_nodes * MC;
    while (word) {
        int p = __ffs(word) - 1;
        word &= word - 1;
        int64_t row = base + nc * 32 + p;
        uint32_t ne = n_edges[row];
        int64_t e0 = edge_index[row];
        for (uint32_t e = 0; e < ne; ++e) {
            uint32_t dst = edge[(e0 + e) * 2];
            uint32_t type = edge[(e0 + e) * 2 + 1];
            for (int j = 0; j < MB; ++j) {
                uint32_t pos = (hv[(int64_t)c * MB + j] + type) % (uint32_t)M;
                uint32_t neg = pos + (uint32_t)M;
                atomicOr(&cx[(int64_t)dst * MC + (pos >> 5)], 1u << (pos & 31));
                atomicAnd(&cx[(int64_t)dst * MC + (neg >> 5)], ~(1u << (neg & 31)));
            }
        }
    }
}

// out[0] |= 1 if on some node a negated literal is not the complement of its positive literal
// (literal k + hv against literal k, hv = literals / 2; bits past the literals are not looked at);
// out[1] |= 1 if some graph has no nodes.  One thread per node, then one per graph.
__global__ void k_graphs_properties(const uint32_t *__restrict__ X, int64_t total_nodes, int LA, int literals,
                                    const uint32_t *__restrict__ n_nodes_arr, int G, uint32_t *out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total_nodes) {
        const uint32_t *row = X + i * LA;
        const int hv = literals / 2;
        bool bad = false;
        if ((hv & 31) == 0) {
            for (int w = 0; w < hv / 32; ++w) bad |= (row[w] ^ row[w + hv / 32]) != 0xFFFFFFFFu;
        } else {
            for (int k = 0; k < hv; ++k) {
                const uint32_t pos = (row[k >> 5] >> (k & 31)) & 1u, neg = (row[(k + hv) >> 5] >> ((k + hv) & 31)) & 1u;
                bad |= pos == neg;
            }
        }
        if (bad) atomicOr(&out[0], 1u);
    }
    if (i < G && n_nodes_arr[i] == 0u) atomicOr(&out[1], 1u);
}

// p[0..n) = v, p[n..total) = 0
__global__ void k_fill_u64(unsigned long long *p, int64_t n, unsigned long long v, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) p[i] = i < n ? v : 0ull;
}

__global__ void k_fill_i32(int32_t *p, int64_t n, int32_t v) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// K6: a block covers TPB clauses of one graph; per class one wave reduction
// and one atomicAdd per wave.
__global__ void k_class_sums(const uint32_t *__restrict__ bitmap, int C, int NC, int K,
                             const int32_t *__restrict__ weights, const uint32_t *__restrict__ n_nodes_arr,
                             int first_graph, int clause_blocks, int32_t *class_sum) {
    int b = blockIdx.x / clause_blocks;
    int c = (blockIdx.x % clause_blocks) * blockDim.x + threadIdx.x;
    int n = (int)n_nodes_arr[first_graph + b];
    bool fired = false;
    if (c < C) {
        int nch = chunks_of(n);
        const uint32_t *row = bitmap + ((int64_t)b * C + c) * NC;
        uint32_t any = 0;
        for (int k = 0; k < nch - 1; ++k) any |= row[k];
        any |= row[nch - 1] & node_filter_of(n);
        fired = any != 0;
    }
    if (__ballot(fired) == 0) return;
    for (int k = 0; k < K; ++k) {
        int v = fired ? weights[(int64_t)k * C + c] : 0;
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
        if ((threadIdx.x & 63) == 0 && v != 0) atomicAdd(&class_sum[(int64_t)b * K + k], v);
    }
}

// K7: uniform choice among the true nodes of each clause.
__global__ void k_select_clause_node(const uint32_t *__restrict__ bitmap, int C, int NC, int n, uint32_t k0, uint32_t k1,
                                     uint32_t step, int32_t *clause_node) {
    int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const uint32_t *row = bitmap + (int64_t)c * NC;
    int nch = n == 0 ? 0 : (n - 1) / 32 + 1;  // an empty graph has no node to pick (kernels.py:336)
    uint32_t last = node_filter_of(n);
    int count = 0;
    for (int k = 0; k < nch; ++k) count += __popc(k == nch - 1 ? row[k] & last : row[k]);
    int node = -1;
    if (count > 0) {
        philox_out r = philox4x32_10((uint32_t)c, 0u, step, GTM_TAG_CLAUSE_NODE, k0, k1);
        int pick = (int)(((uint64_t)r.v[0] * (uint64_t)count) >> 32);
        for (int k = 0; k < nch; ++k) {
            uint32_t w = k == nch - 1 ? row[k] & last : row[k];
            int pc = __popc(w);
            if (pick < pc) {
                for (int j = 0; j < pick; ++j) w &= w - 1;
                node = k * 32 + __ffs(w) - 1;
                break;
            }
            pick -= pc;
        }
    }
    clause_node[c] = node;
}

// K8: feedback decision per (class, clause) and weight update.
__global__ void k_select_clause_updates(int32_t *weights, const int32_t *__restrict__ class_sum,
                                        const int32_t *__restrict__ y, int K, int C, int T, int negative,
                                        uint64_t q_thr, uint32_t k0, uint32_t k1, uint32_t step,
                                        const int32_t *__restrict__ clause_node, int32_t *update) {
    int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    bool fired = clause_node[c] != -1;
    for (int k = 0; k < K; ++k) {
        int cs = class_sum[k];
        cs = cs > T ? T : (cs < -T ? -T : cs);
        int yk = y[k];
        int target = 1 - 2 * (cs > yk);
        int w = weights[(int64_t)k * C + c];
        int sign = (w >= 0) - (w < 0);
        int err = yk - cs;
        err = err < 0 ? -err : err;
        philox_out r = philox4x32_10((uint32_t)c, (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, k0, k1);
        bool skip = (target == -1 && (uint64_t)r.v[0] >= q_thr) ||
                    ((uint64_t)r.v[1] * (uint64_t)(2 * (int64_t)T) >= ((uint64_t)err << 32));
        int u = skip ? 0 : target * sign;
        update[(int64_t)k * C + c] = u;
        if (u > 0 && fired && (w < 0 ? -(int64_t)w : (int64_t)w) < 2147483647) {
            weights[(int64_t)k * C + c] = w + sign;
        } else if (u < 0 && fired) {
            w -= sign;
            if (negative == 0 && w < 1) w = 1;
            weights[(int64_t)k * C + c] = w;
        }
    }
}

#include "fit_fused.h"
#include "fit_deep.h"
#include "fit_small.h"
#include "fit_persistent.h"
#include "fit_deep_persistent.h"

// K9 / K10: one thread per (clause, automaton word); the classes are applied
// in ascending order to that word, as kernels.py:205-207,236-238 do per clause
// (words of a clause do not interact, so splitting by word keeps the result).
__global__ void k_update(uint32_t *bank, int C, int chunks, int B, int K, int boost, int max_included, uint32_t thr16,
                         uint32_t k0, uint32_t k1, uint32_t step, uint32_t bank_id,
                         const int32_t *__restrict__ clause_node, const int32_t *__restrict__ n_incl,
                         const uint32_t *__restrict__ rows, const int32_t *__restrict__ update) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)C * chunks) return;
    int c = (int)(i / chunks), w = (int)(i % chunks);
    int node = clause_node[c];
    bool fired = node != -1;
    bool within = n_incl[c] <= max_included;
    uint32_t x = fired ? rows[(int64_t)node * chunks + w] : 0u;
    uint32_t *ta = bank + i * B;
    feedback_word_any(ta, B, K, update + c, C, fired, within, boost, x, k0, k1, (uint32_t)c, (uint32_t)w, step, bank_id,
                      thr16);
}

// `get_ta_states` / `get_hyperliterals` (kernels.py:718-790): one thread per (clause, literal).
__global__ void k_read_bank(const uint32_t *__restrict__ bank, int C, int chunks, int B, int literals, int actions,
                            uint32_t *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)C * literals) return;
    int c = (int)(i / literals), k = (int)(i % literals);
    const uint32_t *planes = bank + ((int64_t)c * chunks + (k >> 5)) * B;
    uint32_t v;
    if (actions) {
        v = (planes[B - 1] >> (k & 31)) & 1u;
    } else {
        v = 0;
        for (int b = 0; b < B; ++b) v |= ((planes[b] >> (k & 31)) & 1u) << b;
    }
    out[i] = v;
}

// `transform` (kernels.py:671-691): one thread per (graph of the batch, clause).
__global__ void k_transform(const uint32_t *__restrict__ bitmap, int C, int NC,
                            const uint32_t *__restrict__ n_nodes_arr, int first_graph, int64_t total,
                            int32_t *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int b = (int)(i / C);
    int n = (int)n_nodes_arr[first_graph + b];
    const uint32_t *row = bitmap + i * NC;
    uint32_t any = 0;
    if (n > 0) {  // the reference loops over the nodes, so a graph without nodes gives 0
        int chunks = chunks_of(n);
        for (int w = 0; w < chunks - 1; ++w) any |= row[w];
        any |= row[chunks - 1] & node_filter_of(n);
    }
    out[i] = any != 0;
}

// `transform_nodewise` (kernels.py:693-710): one thread per (graph, clause, node < width).
__global__ void k_transform_nodewise(const uint32_t *__restrict__ bitmap, int C, int NC, int width,
                                     const uint32_t *__restrict__ n_nodes_arr, int first_graph, int64_t total,
                                     int32_t *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int node = (int)(i % width);
    int64_t gc = i / width;  // (graph of the batch, clause)
    int n = (int)n_nodes_arr[first_graph + (int)(gc / C)];
    out[i] = node < n ? (bitmap[gc * NC + (node >> 5)] >> (node & 31)) & 1u : 0;
}

// `transform` and `transform_nodewise` (kernels.py:666-710) from the truth rows that the tile kernels
// leave behind ([tiles of the launch][C][tw]), and the class sums (kernels.py:297-315) from the same
// rows: one workgroup per graph.  A graph without nodes gives zeros in both outputs (the reference
// loops over the nodes) while its class sums count every clause, as `evaluate` does.
constexpr int TILE_TRANSFORM_BLOCK = 256;
__global__ __launch_bounds__(TILE_TRANSFORM_BLOCK) void k_tile_transform(
    const uint32_t *__restrict__ bitmap, TileGeom tg, int tile0, int graph0, int first_graph, int C, int K,
    const uint32_t *__restrict__ n_nodes_arr, const int32_t *__restrict__ weights, int32_t *__restrict__ transformed,
    int32_t *__restrict__ nodewise, int width, int32_t *__restrict__ class_sum) {
    extern __shared__ uint32_t fired[];  // one bit per clause, then a partial sum per wave
    int32_t *partial = (int32_t *)(fired + (C + 31) / 32);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = graph0 + (int)blockIdx.x;
    const int n = (int)n_nodes_arr[g];
    const FitGraph f = fit_graph_slot(tg, g, n);
    const uint32_t *rows = bitmap + (int64_t)(f.tile - tile0) * C * tg.tw + f.word0;
    const int64_t out0 = (int64_t)(g - first_graph) * C;
    for (int i = tid; i < (C + 31) / 32; i += TILE_TRANSFORM_BLOCK) fired[i] = 0u;
    __syncthreads();
    for (int c = tid; c < C; c += TILE_TRANSFORM_BLOCK) {
        uint32_t any = 0u;
        for (int w = 0; w < f.words; ++w) any |= (rows[(int64_t)c * tg.tw + w] >> f.shift) & f.mask;
        if (any) atomicOr(&fired[c >> 5], 1u << (c & 31));
        transformed[out0 + c] = n > 0 && any != 0u;
    }
    if (nodewise)
        for (int64_t i = tid; i < (int64_t)C * width; i += TILE_TRANSFORM_BLOCK) {
            const int c = (int)(i / width), node = (int)(i - (int64_t)c * width);
            uint32_t bit = 0u;
            if (node < n) bit = (((rows[(int64_t)c * tg.tw + (node >> 5)] >> f.shift) & f.mask) >> (node & 31)) & 1u;
            nodewise[out0 * width + i] = (int32_t)bit;
        }
    __syncthreads();
    for (int k = 0; k < K; ++k) {
        int sum = 0;
        for (int c = tid; c < C; c += TILE_TRANSFORM_BLOCK)
            if ((fired[c >> 5] >> (c & 31)) & 1u) sum += weights[(int64_t)k * C + c];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
        if (lane == 0) partial[wave] = sum;
        __syncthreads();
        if (tid == 0) {
            int total = 0;
            for (int w = 0; w < TILE_TRANSFORM_BLOCK / 64; ++w) total += partial[w];
            class_sum[(int64_t)(g - first_graph) * K + k] = total;
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------ launch helpers

int launch_clause_node_bits(const Dims &d, const gtm_graphs *g, int first, int n_graphs, const uint32_t *inc_t,
                            int chunks, const uint32_t *rows, int rows_mode, int max_nodes, const uint32_t *cond,
                            uint32_t *out, hipStream_t st) {
    int clause_blocks = (d.C + TPB - 1) / TPB;
    int64_t blocks = (int64_t)clause_blocks * d.NC * n_graphs;
    if (blocks == 0) return GTM_OK;
    if (blocks > 0x7FFFFFFF) return fail(GTM_ERR_INVALID, "batch too large for one launch (%lld blocks)", (long long)blocks);
#define GTM_LAUNCH_CNB(R)                                                                                        \
    hipLaunchKernelGGL((k_clause_node_bits<R>), dim3((unsigned)blocks), dim3(TPB), 0, st, inc_t, d.C, chunks, rows, \
                       rows_mode, max_nodes, g->node_type, g->number_of_node_types, g->node_index,                \
                       g->number_of_graph_nodes, first, d.NC, cond, out, clause_blocks)
    if (chunks <= 2) GTM_LAUNCH_CNB(2);
    else if (chunks <= 4) GTM_LAUNCH_CNB(4);
    else if (chunks <= 8) GTM_LAUNCH_CNB(8);
    else if (chunks <= 16) GTM_LAUNCH_CNB(16);
    else GTM_LAUNCH_CNB(0);
#undef GTM_LAUNCH_CNB
    return check_launch("clause_node_bits");
}

struct Key {
    uint32_t k0, k1;
};
Key key_of(const gtm_config *cfg) { return Key{(uint32_t)(cfg->seed & 0xFFFFFFFFu), (uint32_t)(cfg->seed >> 32)}; }

// Workspace carving -----------------------------------------------------------

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct ScoreWs {
    uint32_t *lists;          // [C][list_stride]  (literal-major tile path)
    int32_t *wt;              // [C][K]
    int list_stride;
    uint32_t *message_lists;  // [depth-1][C][message_list_stride]  (tile path, depth > 1)
    int message_list_stride;
    uint32_t *longest_list;   // [depth-1] entries of each message bank's longest compiled list
    uint32_t *tile_bitmap;    // [tiles per launch][C][tw]  (tile path, depth > 1)
    uint32_t *sent, *got;     // [tiles per launch][tw * 32 node slots][ceil(M / 32)]  (tile path, depth > 1)
    uint32_t *message_rows;   // [tiles per launch][M + 2][tw]  (tile path, depth > 1)
    uint32_t *bit_start, *bit_cursor, *bit_clauses;  // [M + 1], [M], [C * MB]: the clauses of every message bit (tile path, depth > 1)
    uint32_t *alive[2];       // [tiles per launch][streams][alive_stride] clauses still true somewhere in a tile, layer to layer
    uint32_t *stream_order;   // [streams][alive_stride] every clause, by length of its lists (k_narrow_order_keys, _ranks), then [C] keys
    size_t alive_words;       // room per tile
    TileSegment *segments;    // [tiles + 2 * TILE_SEGMENTS_MAX_SHARES] which clauses of which tile a workgroup takes (half tiles)
    size_t vector_words;      // words of sent (and of got)
    uint32_t *inc_t;          // [max(LA,MC)][C]
    uint32_t *bitmap_a;       // [batch][C][NC]
    uint32_t *bitmap_b;       // [batch][C][NC] (depth > 1)
    uint32_t *clause_X;       // [batch][max_nodes][MC] (depth > 1)
    size_t bytes;
};

// Length of a compiled clause: header + type row + literals + what fills its two parts up to whole
// 8-entry blocks, padded to a whole number of 128-entry windows, + 32 entries that a kernel may fetch ahead unused.
int clause_list_stride(int literals) { return ((literals + 2 + 14 + 127) & ~127) + 32; }

// Tiles one launch group covers when the caller asks for `batch` graphs at a time.
int tiles_per_batch(const TileGeom &tg, int batch) { return (batch + tg.gpt - 1) / tg.gpt; }

// `tg`: the data set's tile geometry when the tile path will run (its buffers replace the dense ones).
// `keep_rows` (gtm_transform): the truth rows of the last layer are wanted, also without message layers.
ScoreWs carve_score(const Dims &d, const gtm_config *cfg, int batch, char *base, const TileGeom *tg = nullptr,
                    bool keep_rows = false) {
    ScoreWs w{};
    size_t off = 0;
    int chunks = cfg->depth > 1 && d.MC > d.LA ? d.MC : d.LA;
    auto take = [&](size_t bytes) {
        char *p = base ? base + off : nullptr;
        off += align_up(bytes);
        return p;
    };
    w.list_stride = clause_list_stride(cfg->literals);
    w.lists = (uint32_t *)take((size_t)d.C * w.list_stride * 4);
    w.wt = (int32_t *)take((size_t)d.C * d.K * 4);
    // (+ a key per clause after the table)
    if (tg) w.stream_order = (uint32_t *)take((2 * (size_t)d.C + 2 * NARROW_MAX_STREAMS) * 4);
    if (tg && cfg->depth == 1 && tg->half)
        w.segments = (TileSegment *)take(((size_t)tg->n_tiles + 2 * TILE_SEGMENTS_MAX_SHARES) * sizeof(TileSegment));
    if (tg && cfg->depth == 1 && !keep_rows) {
        w.bytes = off;
        return w;
    }
    if (tg && cfg->depth == 1) {
        w.tile_bitmap = (uint32_t *)take((size_t)tiles_per_batch(*tg, batch) * d.C * tg->tw * 4);
        w.bytes = off;
        return w;
    }
    if (tg) {
        w.message_list_stride = clause_list_stride(2 * d.M);
        w.message_lists = (uint32_t *)take((size_t)(cfg->depth - 1) * d.C * w.message_list_stride * 4);
        w.longest_list = (uint32_t *)take((size_t)(cfg->depth - 1) * 4);
        const size_t n_tiles = tiles_per_batch(*tg, batch);
        w.tile_bitmap = (uint32_t *)take(n_tiles * d.C * tg->tw * 4);
        w.vector_words = n_tiles * tg->tw * 32 * ((d.M + 31) / 32);
        w.sent = (uint32_t *)take(w.vector_words * 4);
        w.got = (uint32_t *)take(w.vector_words * 4);
        w.message_rows = (uint32_t *)take(n_tiles * tile_message_rows(d.M) * tg->tw * 4);
        w.bit_start = (uint32_t *)take(((size_t)d.M + 1) * 4);
        w.bit_cursor = (uint32_t *)take((size_t)d.M * 4);
        w.bit_clauses = (uint32_t *)take((size_t)d.C * d.MB * 4);
        // (per tile: `streams` lists of 1 + ceil(C / streams) words, whichever shape k_tile_layer_narrow takes)
        w.alive_words = (size_t)d.C + 2 * NARROW_MAX_STREAMS;
        for (uint32_t *&list : w.alive) list = (uint32_t *)take(n_tiles * w.alive_words * 4);
        w.bytes = off;
        return w;
    }
    w.inc_t = (uint32_t *)take((size_t)chunks * d.C * 4);
    w.bitmap_a = (uint32_t *)take((size_t)batch * d.C * d.NC * 4);
    if (cfg->depth > 1) {
        w.bitmap_b = (uint32_t *)take((size_t)batch * d.C * d.NC * 4);
        w.clause_X = (uint32_t *)take((size_t)batch * cfg->max_nodes * d.MC * 4);
    }
    w.bytes = off;
    return w;
}

struct FitWs {
    uint32_t *inc_t;
    uint32_t *bitmap_a, *bitmap_b;
    uint32_t *clause_X[GTM_MAX_DEPTH - 1];  // per message layer, kept for K10
    int32_t *class_sum;                     // [K]
    int32_t *clause_node;                   // [C]
    int32_t *n_incl;                        // [C]
    int32_t *update;                        // [K][C]
    uint32_t *message_rows;                 // [M][message_row_words] literal-major messages of one layer (depth > 1)
    int message_row_words;
    uint32_t *sent, *got;                   // [max_nodes][M / 32] bit vectors sent / received per node (depth > 1)
    uint32_t *bank_backup;                  // every bank as it was before a cooperative run: [C][LA][B], then [C][MC][B] per message bank
    int32_t *weights_backup;                // [K][C]
    uint32_t *coop_got;                     // [3][depth - 1][M][NC] rows exchanged by k_fit_deep_persistent (depth > 1)
    uint32_t *coop_vec;                     // [depth - 1][max_nodes][M / 32] the same, node-major
    unsigned long long *coop_arrived;       // [depth - 1][FITD_PARTS * FITD_STRIDE]
    size_t coop_words;                      // words of coop_got
    int *coop_perm;                         // [C + 2,048] which clause sits in which workgroup's slots (k_fit_deep_deal)
    uint32_t *coop_cost;                    // [C]
    size_t bytes;
};

FitWs carve_fit(const Dims &d, const gtm_config *cfg, char *base) {
    FitWs w;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char *p = base ? base + off : nullptr;
        off += align_up(bytes);
        return p;
    };
    int chunks = cfg->depth > 1 && d.MC > d.LA ? d.MC : d.LA;
    w.inc_t = (uint32_t *)take((size_t)chunks * d.C * 4);
    w.bitmap_a = (uint32_t *)take((size_t)d.C * d.NC * 4);
    w.bitmap_b = (uint32_t *)take((size_t)d.C * d.NC * 4);
    for (int l = 0; l < GTM_MAX_DEPTH - 1; ++l)
        w.clause_X[l] = l < cfg->depth - 1 ? (uint32_t *)take((size_t)cfg->max_nodes * d.MC * 4) : nullptr;
    // the fused paths rotate class-sum buffers: 2 x int32 [K], or 3 x 64-bit [K] followed by an abort flag
    w.class_sum = (int32_t *)take(((size_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE + 1) * 8);  // the persistent kernel's ring is the largest user
    w.clause_node = (int32_t *)take((size_t)d.C * 4);
    w.n_incl = (int32_t *)take((size_t)d.C * 4);
    w.update = (int32_t *)take((size_t)d.K * d.C * 4);
    w.message_row_words = 2 * ((cfg->max_nodes + 63) / 64);
    w.message_rows = cfg->depth > 1 ? (uint32_t *)take((size_t)d.M * w.message_row_words * 4) : nullptr;
    const size_t vector_bytes = (size_t)cfg->max_nodes * ((d.M + 31) / 32) * 4;
    w.sent = cfg->depth > 1 ? (uint32_t *)take(vector_bytes) : nullptr;
    w.got = cfg->depth > 1 ? (uint32_t *)take(vector_bytes) : nullptr;
    w.bank_backup = (uint32_t *)take(((size_t)d.C * d.LA + (size_t)(cfg->depth - 1) * d.C * d.MC) * d.B * 4);
    w.weights_backup = (int32_t *)take((size_t)d.K * d.C * 4);
    w.coop_words = cfg->depth > 1 ? (size_t)3 * (cfg->depth - 1) * d.M * d.NC : 0;
    w.coop_got = cfg->depth > 1 ? (uint32_t *)take(w.coop_words * 4) : nullptr;
    w.coop_vec = cfg->depth > 1 ? (uint32_t *)take((size_t)(cfg->depth - 1) * cfg->max_nodes * d.MC * 2) : nullptr;
    w.coop_arrived = cfg->depth > 1 ? (unsigned long long *)take((size_t)(cfg->depth - 1) * FITD_PARTS * FITD_STRIDE * 8) : nullptr;
    w.coop_perm = cfg->depth > 1 ? (int *)take(((size_t)d.C + 2048) * 4) : nullptr;
    w.coop_cost = cfg->depth > 1 ? (uint32_t *)take((size_t)d.C * 4) : nullptr;
    w.bytes = off;
    return w;
}

// Operator bodies shared by the per-kernel entry points and the driver loops ----

int op_include_plane(const Dims &d, const uint32_t *bank, int chunks, uint32_t filter, uint32_t *inc_t, int32_t *n_incl,
                     int accumulate, hipStream_t st) {
    hipLaunchKernelGGL(k_include_plane, dim3(blocks_for(d.C, TPB)), dim3(TPB), 0, st, bank, d.C, chunks, d.B, filter,
                       inc_t, n_incl, accumulate);
    return check_launch("include_plane");
}

int op_exchange(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, int first, int n_graphs,
                const uint32_t *hv, const uint32_t *bitmap, uint32_t *clause_X, hipStream_t st) {
    if (n_graphs == 0) return GTM_OK;
    int64_t words = (int64_t)n_graphs * cfg->max_nodes * d.MC;
    hipLaunchKernelGGL(k_messages_blank, dim3(blocks_for(words, TPB)), dim3(TPB), 0, st, clause_X, words, d.MC, d.M);
    if (int rc = check_launch("messages_blank")) return rc;
    if (g->total_edges > 0) {
        if (!g->number_of_graph_node_edges || !g->edge || !g->edge_index)
            return fail(GTM_ERR_INVALID, "graphs with edges need number_of_graph_node_edges, edge and edge_index");
        int64_t total = (int64_t)n_graphs * d.C * d.NC;
        hipLaunchKernelGGL(k_messages_scatter, dim3(blocks_for(total, TPB)), dim3(TPB), 0, st, bitmap, d.C, d.NC, hv,
                           d.MB, d.M, d.MC, cfg->max_nodes, g->node_index, g->number_of_graph_nodes,
                           g->number_of_graph_node_edges, g->edge_index, g->edge, first, total, clause_X);
        if (int rc = check_launch("messages_scatter")) return rc;
    }
    return GTM_OK;
}

int op_class_sums(const Dims &d, const gtm_graphs *g, int first, int n_graphs, const uint32_t *bitmap,
                  const int32_t *weights, int32_t *class_sum, hipStream_t st) {
    if (n_graphs == 0) return GTM_OK;
    int64_t n = (int64_t)n_graphs * d.K;
    hipLaunchKernelGGL(k_fill_i32, dim3(blocks_for(n, TPB)), dim3(TPB), 0, st, class_sum, n, 0);
    if (int rc = check_launch("fill")) return rc;
    int clause_blocks = (d.C + TPB - 1) / TPB;
    hipLaunchKernelGGL(k_class_sums, dim3((unsigned)(clause_blocks * (int64_t)n_graphs)), dim3(TPB), 0, st, bitmap, d.C,
                       d.NC, d.K, weights, g->number_of_graph_nodes, first, clause_blocks, class_sum);
    return check_launch("class_sums");
}

// The graph-independent part of `_evaluate` for a batch (tm.py:563-662).
// Leaves the final bitmap in *final_bitmap.
int run_evaluate(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, int first, int n_graphs,
                 uint32_t *inc_t, uint32_t *bm_a, uint32_t *bm_b, uint32_t *const *clause_X, bool keep_layers,
                 int32_t *n_incl, int32_t *class_sum, uint32_t **final_bitmap, hipStream_t st) {
    if (int rc = op_include_plane(d, s->ta_state, d.LA, d.filter, inc_t, n_incl, 0, st)) return rc;
    profile_start("k_clause_node_bits", st);
    if (int rc = launch_clause_node_bits(d, g, first, n_graphs, inc_t, d.LA, g->X, 0, cfg->max_nodes, nullptr, bm_a, st))
        return rc;
    profile_stop(st);
    uint32_t *cur = bm_a, *nxt = bm_b;
    for (int layer = 0; layer < cfg->depth - 1; ++layer) {
        uint32_t *cx = keep_layers ? clause_X[layer] : clause_X[0];
        if (int rc = op_exchange(d, cfg, g, first, n_graphs, s->hypervectors, cur, cx, st)) return rc;
        if (int rc = op_include_plane(d, s->message_ta_state[layer], d.MC, d.mfilter, inc_t, n_incl, 1, st)) return rc;
        if (int rc = launch_clause_node_bits(d, g, first, n_graphs, inc_t, d.MC, cx, 1, cfg->max_nodes, cur, nxt, st))
            return rc;
        uint32_t *t = cur;
        cur = nxt;
        nxt = t;
    }
    if (int rc = op_class_sums(d, g, first, n_graphs, cur, s->clause_weights, class_sum, st)) return rc;
    *final_bitmap = cur;
    return GTM_OK;
}

int validate_state(const gtm_config *cfg, const gtm_state *s) {
    if (!s) return fail(GTM_ERR_INVALID, "state is NULL");
    if (!s->ta_state || !s->clause_weights) return fail(GTM_ERR_INVALID, "state has NULL ta_state or clause_weights");
    for (int l = 0; l < cfg->depth - 1; ++l)
        if (!s->message_ta_state[l]) return fail(GTM_ERR_INVALID, "state lacks message_ta_state[%d]", l);
    if (cfg->depth > 1 && !s->hypervectors) return fail(GTM_ERR_INVALID, "state lacks hypervectors");
    return GTM_OK;
}

// Words of bit rows in a tile buffer, padded so that the row counts after them are 8-byte aligned.
size_t tiles_words(const TileGeom &tg) { return ((size_t)tg.n_tiles * tg.rows * tg.tw + 1) & ~(size_t)1; }

// Half tiles carry a fourth part after the rows, the row counts and the literal order: the positive
// half of every node's literal words, by node SLOT ([tile][slot of the tile][LA / 2] words, zeros in
// slots without a node), 16-byte aligned.  Phase 2 of k_tile_two_phase_half reads it instead of X:
// half the bytes per candidate node, no lookup of the graph's first node, and a tile's share of it
// stays in the XCD's L2 while the tile's clauses are worked through.
size_t tiles_xpos_offset_words(const TileGeom &tg, int literals) {
    return (tiles_words(tg) + (size_t)tg.rows * 2 + (size_t)literals + 3) & ~(size_t)3;
}
size_t tiles_xpos_words(const TileGeom &tg, int literals) {
    return tg.half ? (size_t)tg.n_tiles * tg.tw * 32 * (size_t)(literals / 64) : 0;
}

// Inference on literal-major tiles (see score_tiles.h).
int max_lane_words() {
    const char *e = tune(T_TILE_LANE_WORDS);  // 1, 2 or 4: upper bound on words per lane (tuning aid)
    int v = e ? atoi(e) : 4;
    return v == 1 || v == 2 ? v : 4;
}

// Half tiles (positive rows only in LDS, k_tile_two_phase_half): a depth-1 model on a data set that
// the caller has declared complementary, with word-aligned halves of 4 to 16 literal words per node.
// GTM_NO_HALF_TILES (tuning aid) turns them off.  (The kernel reads the weights at 32-bit byte offsets.)
bool half_tiles_allowed(const gtm_config *cfg, const gtm_graphs *g) {
    const int LA = (cfg->literals - 1) / 32 + 1;
    return cfg->depth == 1 && (g->flags & GTM_GRAPHS_COMPLEMENTARY) && cfg->literals % 64 == 0 && LA % 4 == 0 &&
           LA <= 16 && (int64_t)cfg->clauses * cfg->classes < (1 << 28) && !tune(T_NO_HALF_TILES) && !tune(T_NO_TWO_PHASE);
}

TileGeom geometry_for(const gtm_config *cfg, const gtm_graphs *g, int classes) {
    return tile_geometry(cfg->literals, g->number_of_node_types, g->max_number_of_graph_nodes, g->number_of_graphs,
                         classes, max_lane_words(), cfg->depth > 1 ? tile_message_rows(cfg->message_size) : 0,
                         half_tiles_allowed(cfg, g), tune(T_HALF_LANE_WORDS) ? atoi(tune(T_HALF_LANE_WORDS)) : 0);
}

// The geometry every tile buffer of this process was built for, by address.  The driver loops
// recompute the geometry from their arguments on every call; a buffer built for other arguments
// (another number of classes, depth, message size or lane-width setting) would be read with the
// wrong row width, so such a call is refused.  (Leaked on purpose: no destructor runs at exit.)
struct TilesTag {
    TileGeom tg;
    int literals, n_types, n_graphs;
};
std::mutex g_tiles_mutex;
std::unordered_map<const void *, TilesTag> &tiles_registry() {
    static auto *m = new std::unordered_map<const void *, TilesTag>();
    return *m;
}

void remember_tiles(const void *tiles, const TileGeom &tg, const gtm_config *cfg, const gtm_graphs *g) {
    std::lock_guard<std::mutex> lock(g_tiles_mutex);
    tiles_registry()[tiles] = TilesTag{tg, cfg->literals, g->number_of_node_types, g->number_of_graphs};
}

int check_tiles(const TileGeom &tg, const gtm_config *cfg, const gtm_graphs *g) {
    std::lock_guard<std::mutex> lock(g_tiles_mutex);
    auto it = tiles_registry().find(g->tiles);
    if (it == tiles_registry().end())
        return fail(GTM_ERR_INVALID, "graphs->tiles was not filled by gtm_build_tiles in this process");
    const TilesTag &t = it->second;
    if (memcmp(&t.tg, &tg, sizeof tg) != 0 || t.literals != cfg->literals || t.n_types != g->number_of_node_types ||
        t.n_graphs != g->number_of_graphs)
        return fail(GTM_ERR_INVALID,
                    "graphs->tiles was built for another configuration (rows of %d words x %d rows, %d graphs per "
                    "tile; this call needs %d x %d, %d): build the tiles again with this configuration",
                    t.tg.tw, t.tg.rows, t.tg.gpt, tg.tw, tg.rows, tg.gpt);
    return GTM_OK;
}

// Workgroups that share a tile's clauses when layer 0 reads its rows in place and the tiles are few.
int tile_layer_splits(const TileLayerArgs &a, int n_tiles, int src) {
    if (src != ROWS_GLOBAL) return 1;
    int splits = (512 + n_tiles - 1) / n_tiles;
    const int most = (a.C + 15) / 16;  // at least one clause per wave
    splits = splits > most ? most : splits;
    return splits < 1 ? 1 : splits > 64 ? 64 : splits;
}

template <int NW, int LW, int SRC, bool LAST>
int launch_tile_layer_as(const TileLayerArgs &a_in, int n_tiles, const char *profile_name, hipStream_t st) {
    TileLayerArgs a = a_in;
    size_t lds = tile_layer_lds_bytes(a.tg, a.K, SRC, a.M);
    // message layers: room for every wave's clause list where LDS has it (GTM_NO_LISTS_IN_LDS: tuning and test aid)
    a.lists_in_lds = 0;
    if (SRC == ROWS_MESSAGES && lds + (size_t)NW * TILE_LIST_LDS_WORDS * 4 <= 160 * 1024 && !tune(T_NO_LISTS_IN_LDS)) {
        a.lists_in_lds = 1;
        lds += (size_t)NW * TILE_LIST_LDS_WORDS * 4;
    }
    const int splits = tile_layer_splits(a, n_tiles, SRC);
    if (LAST && splits > 1) {  // the workgroups of a tile add their shares
        const int64_t n = (int64_t)a.n_graphs * a.K;
        hipLaunchKernelGGL(k_fill_i32, dim3(blocks_for(n, TPB)), dim3(TPB), 0, st, a.class_sum, n, 0);
        if (int rc = check_launch("fill")) return rc;
    }
    static thread_local size_t lds_set = 48 * 1024;
    if (lds > lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)k_tile_layer<NW, LW, SRC, LAST>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
        lds_set = lds;
    }
    if (profile_name) profile_start(profile_name, st);
    hipLaunchKernelGGL((k_tile_layer<NW, LW, SRC, LAST>), dim3(n_tiles, splits), dim3(NW * 64), lds, st, a);
    if (int rc = check_launch("tile_layer")) return rc;
    if (profile_name) profile_stop(st);
    return GTM_OK;
}

template <int NW, int LW>
int launch_tile_layer_lw(const TileLayerArgs &a, int n_tiles, int src, bool last, hipStream_t st) {
    if (src == ROWS_MESSAGES)
        return last ? launch_tile_layer_as<NW, LW, ROWS_MESSAGES, true>(a, n_tiles, "k_tile_layer<messages, score>", st)
                    : launch_tile_layer_as<NW, LW, ROWS_MESSAGES, false>(a, n_tiles, "k_tile_layer<messages>", st);
    if (src == ROWS_GLOBAL)
        return last ? launch_tile_layer_as<NW, LW, ROWS_GLOBAL, true>(a, n_tiles, "k_tile_layer<score>", st)
                    : launch_tile_layer_as<NW, LW, ROWS_GLOBAL, false>(a, n_tiles, "k_tile_layer<layer0>", st);
    return last ? launch_tile_layer_as<NW, LW, ROWS_STAGED, true>(a, n_tiles, "k_tile_layer<score>", st)
                : launch_tile_layer_as<NW, LW, ROWS_STAGED, false>(a, n_tiles, "k_tile_layer<layer0>", st);
}

int launch_tile_layer(const TileLayerArgs &a, int n_tiles, int src, bool last, hipStream_t st) {
    constexpr int NW = 16;
    switch (a.tg.lw) {
        case 1: return launch_tile_layer_lw<NW, 1>(a, n_tiles, src, last, st);
        case 2: return launch_tile_layer_lw<NW, 2>(a, n_tiles, src, last, st);
        default: return launch_tile_layer_lw<NW, 4>(a, n_tiles, src, last, st);
    }
}

template <int NW, int LW, int LA4, bool LAST, bool FULL>
int launch_two_phase_as(const TileLayerArgs &a, int n_tiles, hipStream_t st) {
    size_t lds = tile_layer_lds_bytes(a.tg, a.K, ROWS_STAGED, a.M);
    static thread_local size_t lds_set = 48 * 1024;
    if (lds > lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)k_tile_two_phase<NW, LW, LA4, LAST, FULL>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
        lds_set = lds;
    }
    profile_start(LAST ? "k_tile_two_phase<score>" : "k_tile_two_phase<layer0>", st);
    hipLaunchKernelGGL((k_tile_two_phase<NW, LW, LA4, LAST, FULL>), dim3(n_tiles), dim3(NW * 64), lds, st, a);
    if (int rc = check_launch("tile_two_phase")) return rc;
    profile_stop(st);
    return GTM_OK;
}

template <int NW, int LW, int LA4>
int launch_two_phase_la(const TileLayerArgs &a, int n_tiles, bool last, hipStream_t st) {
    const bool full = a.tg.tw == 64 * LW;
    if (last)
        return full ? launch_two_phase_as<NW, LW, LA4, true, true>(a, n_tiles, st)
                    : launch_two_phase_as<NW, LW, LA4, true, false>(a, n_tiles, st);
    return full ? launch_two_phase_as<NW, LW, LA4, false, true>(a, n_tiles, st)
                : launch_two_phase_as<NW, LW, LA4, false, false>(a, n_tiles, st);
}

template <int NW, int LW>
int launch_two_phase_lw(const TileLayerArgs &a, int n_tiles, int la4, bool last, hipStream_t st) {
    switch (la4) {
        case 1: return launch_two_phase_la<NW, LW, 1>(a, n_tiles, last, st);
        case 2: return launch_two_phase_la<NW, LW, 2>(a, n_tiles, last, st);
        case 3: return launch_two_phase_la<NW, LW, 3>(a, n_tiles, last, st);
        default: return launch_two_phase_la<NW, LW, 4>(a, n_tiles, last, st);
    }
}

int launch_two_phase(const TileLayerArgs &a, int n_tiles, int la4, bool last, hipStream_t st) {
    constexpr int NW = 16;
    switch (a.tg.lw) {
        case 1: return launch_two_phase_lw<NW, 1>(a, n_tiles, la4, last, st);
        case 2: return launch_two_phase_lw<NW, 2>(a, n_tiles, la4, last, st);
        default: return launch_two_phase_lw<NW, 4>(a, n_tiles, la4, last, st);
    }
}

// Compute units of the current device (0 if it cannot be told).
int compute_units() {
    static thread_local int cus_of[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cus_of[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        cus_of[dev] = cus;
    }
    return cus_of[dev];
}

// The tiles of a launch of k_tile_two_phase_half shared out among the compute units (tile_segments_part
// in score_tiles.h) - when they do not fill a whole number of rounds of the chip, and a share is at least 64
// clauses (a share stages its tile).  GTM_NO_TILE_LINE turns it off; GTM_TILE_LINE_GROUPS = n (tests) cuts the
// tiles into n shares whatever the device has.  cus == 0 in the result: one workgroup per tile.
SegmentPlan plan_segments(const TileLayerArgs &a, int n_tiles, TileSegment *segments) {
    SegmentPlan sp{};
    int cus = compute_units();
    bool shared_out = cus > 0 && n_tiles % cus != 0 && (int64_t)(n_tiles % cus) * a.C / cus >= 64 && !tune(T_NO_TILE_LINE);
    if (const char *e = tune(T_TILE_LINE_GROUPS)) {
        cus = atoi(e);
        shared_out = cus >= 1;
    }
    // (the table's arithmetic is 32-bit; a block of the compile launch holds at most 16 waves)
    if (!shared_out || !segments || cus > TILE_SEGMENTS_MAX_SHARES || (int64_t)(n_tiles % cus) * a.C >= (1ll << 31)) return sp;
    sp.n_tiles = n_tiles, sp.C = a.C, sp.cus = cus, sp.gpt = a.tg.gpt, sp.K = a.K, sp.tile0 = a.tile0;
    sp.first_graph = a.first_graph, sp.n_graphs = a.n_graphs, sp.segments = segments, sp.class_sum = a.class_sum;
    return sp;
}

template <int NW, int LW, int LA4, bool LAST, bool FULL>
int launch_two_phase_half_as(const TileLayerArgs &a_in, int n_tiles, const SegmentPlan *sp, hipStream_t st) {
    TileLayerArgs a = a_in;
    const bool shared_out = LAST && sp && sp->cus > 0;
    a.segments = shared_out ? sp->segments : nullptr;
    const int groups = shared_out ? tile_segment_count(n_tiles, sp->cus) : n_tiles;
    const size_t lds = tile_lds_bytes(a.tg.rows - LA4 * 64, a.tg, a.K);  // the rows of the negated literals stay out
    static thread_local size_t lds_set = 48 * 1024;
    if (lds > lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)k_tile_two_phase_half<NW, LW, LA4, LAST, FULL>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
        lds_set = lds;
    }
    profile_start(LAST ? "k_tile_two_phase_half<score>" : "k_tile_two_phase_half<layer0>", st);
    hipLaunchKernelGGL((k_tile_two_phase_half<NW, LW, LA4, LAST, FULL>), dim3(groups), dim3(NW * 64), lds, st, a);
    if (int rc = check_launch("tile_two_phase_half")) return rc;
    profile_stop(st);
    return GTM_OK;
}

template <int NW, int LW, int LA4>
int launch_two_phase_half_la(const TileLayerArgs &a, int n_tiles, bool last, const SegmentPlan *segments, hipStream_t st) {
    const bool full = a.tg.tw == 64 * LW;
    if (last)
        return full ? launch_two_phase_half_as<NW, LW, LA4, true, true>(a, n_tiles, segments, st)
                    : launch_two_phase_half_as<NW, LW, LA4, true, false>(a, n_tiles, segments, st);
    return full ? launch_two_phase_half_as<NW, LW, LA4, false, true>(a, n_tiles, segments, st)
                : launch_two_phase_half_as<NW, LW, LA4, false, false>(a, n_tiles, segments, st);
}

template <int NW, int LW>
int launch_two_phase_half_lw(const TileLayerArgs &a, int n_tiles, int la4, bool last, const SegmentPlan *segments, hipStream_t st) {
    switch (la4) {
        case 1: return launch_two_phase_half_la<NW, LW, 1>(a, n_tiles, last, segments, st);
        case 2: return launch_two_phase_half_la<NW, LW, 2>(a, n_tiles, last, segments, st);
        case 3: return launch_two_phase_half_la<NW, LW, 3>(a, n_tiles, last, segments, st);
        default: return launch_two_phase_half_la<NW, LW, 4>(a, n_tiles, last, segments, st);
    }
}

int launch_two_phase_half(const TileLayerArgs &a, int n_tiles, int la4, bool last, const SegmentPlan *segments, hipStream_t st) {
    constexpr int NW = 16;
    switch (a.tg.lw) {
        case 1: return launch_two_phase_half_lw<NW, 1>(a, n_tiles, la4, last, segments, st);
        case 2: return launch_two_phase_half_lw<NW, 2>(a, n_tiles, la4, last, segments, st);
        default: return launch_two_phase_half_lw<NW, 4>(a, n_tiles, la4, last, segments, st);
    }
}

template <int NW, int LW, int SRC, bool LAST>
int launch_two_phase_wide_as(const TileLayerArgs &a, int n_tiles, int LA, hipStream_t st) {
    // rows (if staged), padding, class sums, and the first node and node count of the tile's graphs
    // several narrow tiles per wave (rows read in place, truth rows only, one word per lane): see the kernel
    int pack = 1;
    if (SRC == ROWS_GLOBAL && !LAST && LW == 1 && a.tg.tw <= 32 && !tune(T_NO_TILE_PACK))
        pack = 64 / a.tg.tw;
    const int n_groups = (n_tiles + pack - 1) / pack;
    size_t lds = tile_layer_lds_bytes(a.tg, a.K, SRC, a.M) + (size_t)pack * a.tg.gpt * 8;
    static thread_local size_t lds_set = 48 * 1024;
    if (lds > lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)k_tile_two_phase_wide<NW, LW, SRC, LAST>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
        lds_set = lds;
    }
    // rows read in place and no votes: several workgroups share a tile's clauses until the chip is full
    int splits = 1;
    if (SRC == ROWS_GLOBAL && !LAST) {
        splits = 2048 / (n_groups > 0 ? n_groups : 1);
        splits = splits < 1 ? 1 : (splits > 16 ? 16 : splits);
        if (const char *e = tune(T_WIDE_SPLITS)) splits = std::max(1, std::min(64, atoi(e)));
    }
    profile_start(LAST ? "k_tile_two_phase_wide<score>" : "k_tile_two_phase_wide<layer0>", st);
    hipLaunchKernelGGL((k_tile_two_phase_wide<NW, LW, SRC, LAST>), dim3((unsigned)((n_groups + 7) / 8 * 8 * splits)),
                       dim3(NW * 64), lds, st, a, LA, n_tiles, splits, pack);
    if (int rc = check_launch("tile_two_phase_wide")) return rc;
    profile_stop(st);
    return GTM_OK;
}

template <int NW, int LW>
int launch_two_phase_wide_lw(const TileLayerArgs &a, int n_tiles, int LA, bool staged, bool last, hipStream_t st) {
    if (staged)
        return last ? launch_two_phase_wide_as<NW, LW, ROWS_STAGED, true>(a, n_tiles, LA, st)
                    : launch_two_phase_wide_as<NW, LW, ROWS_STAGED, false>(a, n_tiles, LA, st);
    return last ? launch_two_phase_wide_as<NW, LW, ROWS_GLOBAL, true>(a, n_tiles, LA, st)
                : launch_two_phase_wide_as<NW, LW, ROWS_GLOBAL, false>(a, n_tiles, LA, st);
}

int launch_two_phase_wide(const TileLayerArgs &a, int n_tiles, int LA, bool staged, bool last, hipStream_t st) {
    constexpr int NW = 16;
    switch (a.tg.lw) {
        case 1: return launch_two_phase_wide_lw<NW, 1>(a, n_tiles, LA, staged, last, st);
        case 2: return launch_two_phase_wide_lw<NW, 2>(a, n_tiles, LA, staged, last, st);
        default: return launch_two_phase_wide_lw<NW, 4>(a, n_tiles, LA, staged, last, st);
    }
}

// Several clauses per wave on narrow tiles (score_narrow.h).
template <int SRC, bool LAST, int GROUP, int WPL>
int launch_narrow_as(const TileLayerArgs &a, const NarrowArgs &x, int n_tiles, hipStream_t st) {
    const size_t lds = narrow_lds_bytes(a.tg, NarrowChoice{GROUP, WPL}, a.K, narrow_rows_lds(SRC, a.M, x.hv, x.n_types), x.row_words);
    static thread_local size_t lds_set = 48 * 1024;
    if (lds > lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)k_tile_layer_narrow<SRC, LAST, GROUP, WPL>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
        lds_set = lds;
    }
    profile_start(SRC == ROWS_HALF ? (LAST ? "k_tile_layer_narrow<score>" : "k_tile_layer_narrow<layer0>")
                                   : (LAST ? "k_tile_layer_narrow<messages, score>" : "k_tile_layer_narrow<messages>"),
                  st);
    hipLaunchKernelGGL((k_tile_layer_narrow<SRC, LAST, GROUP, WPL>), dim3(n_tiles), dim3(NARROW_WAVES * 64), lds, st, a, x);
    if (int rc = check_launch("tile_layer_narrow")) return rc;
    profile_stop(st);
    return GTM_OK;
}

template <int GROUP, int WPL>
int launch_narrow_shape(const TileLayerArgs &a, const NarrowArgs &x, int n_tiles, int src, bool last, hipStream_t st) {
    if (src == ROWS_HALF)
        return last ? launch_narrow_as<ROWS_HALF, true, GROUP, WPL>(a, x, n_tiles, st)
                    : launch_narrow_as<ROWS_HALF, false, GROUP, WPL>(a, x, n_tiles, st);
    return last ? launch_narrow_as<ROWS_MESSAGES, true, GROUP, WPL>(a, x, n_tiles, st)
                : launch_narrow_as<ROWS_MESSAGES, false, GROUP, WPL>(a, x, n_tiles, st);
}

int launch_narrow(const TileLayerArgs &a, const NarrowArgs &x, const NarrowChoice &shape, int n_tiles, int src, bool last,
                  hipStream_t st) {
    if (shape.group == 8 && shape.wpl == 4) return launch_narrow_shape<8, 4>(a, x, n_tiles, src, last, st);
    if (shape.group == 16 && shape.wpl == 4) return launch_narrow_shape<16, 4>(a, x, n_tiles, src, last, st);
    if (shape.group == 16 && shape.wpl == 2) return launch_narrow_shape<16, 2>(a, x, n_tiles, src, last, st);
    return fail(GTM_ERR_INVALID, "no narrow-tile kernel for %d lanes per clause and %d words per lane", shape.group, shape.wpl);
}

// Layer 0 can run in two phases (k_tile_two_phase) on tiles of whole-word graph slots staged in
// LDS when a node has 4, 8, 12 or 16 literal words.  GTM_NO_TWO_PHASE (tuning aid) turns it off.
bool two_phase_layer0(const Dims &d, const gtm_graphs *g, const TileGeom &tg) {
    if (tg.half) return true;  // such a geometry is only chosen for k_tile_two_phase_half (64-bit offsets into X)
    // k_tile_two_phase addresses X with 32-bit byte offsets: beyond 4 GiB of literal words (or with
    // GTM_NO_NARROW_TWO_PHASE, which lets tests take that way with small data) k_tile_two_phase_wide runs
    const bool x_fits = (uint64_t)g->total_nodes * d.LA * 4 < (1ull << 32) && !tune(T_NO_NARROW_TWO_PHASE);
    return tg.slot_words > 0 && tg.stage0 && d.LA % 4 == 0 && d.LA <= 16 && x_fits && !tune(T_NO_TWO_PHASE);
}

// `_score`'s loop (tm.py:786-812) on tiles: per launch group of tiles, layer 0 and then one
// launch per message layer; the clause truth rows between layers stay in w.tile_bitmap.
// With `tr` (gtm_transform; tm.py:814-900) every layer leaves its truth rows, and k_tile_transform
// makes the per-clause outputs and the class sums from the last layer's.
struct TransformOut {
    int32_t *transformed, *nodewise;
    int width;
};

int score_on_tiles(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, const TileGeom &tg,
                   const ScoreWs &w, int first, int n_graphs, int batch, int32_t *class_sum, hipStream_t st,
                   const TransformOut *tr = nullptr) {
    const uint32_t *order = g->tiles + tiles_words(tg) + (size_t)tg.rows * 2;
    const int layers = cfg->depth;
    const bool narrow = two_phase_layer0(d, g, tg);
    // any other tile of whole-word slots whose row offsets fit the 16-bit entries: k_tile_two_phase_wide
    const bool wide = !narrow && tg.slot_words > 0 && (int64_t)tg.rows * tg.tw / 4 < 65536 && !tune(T_NO_TWO_PHASE);
    const bool two_phase = narrow || wide;
    // Narrow tiles: four clauses per wave (score_narrow.h) for the message layers, and for layer 0 when the data
    // set's negated literals are the complements of its positive ones, so that the positive rows alone, which
    // fit in LDS, will do.  GTM_NO_NARROW_LAYERS / GTM_NO_HALF_ROWS (tuning and test aids) turn them off.
    const size_t lds_limit = 160 * 1024;
    const int hv = cfg->literals / 2;
    // (GTM_NARROW_READS=128, tuning and test aid: rows of at most 32 words on 128-bit reads, eight clauses per wave)
    const char *narrow_reads = tune(T_NARROW_READS);
    const NarrowChoice shape = narrow_choice(tg, narrow_reads && atoi(narrow_reads) == 128);
    // (the kernel reaches lists and truth rows at 32-bit byte offsets formed from 24-bit factors)
    const bool narrow_tiles = shape.group != 0 && !tune(T_NO_NARROW_LAYERS) && d.C < (1 << 24) && (int64_t)d.C * d.K < (1 << 28) &&
                              (int64_t)d.C * std::max(w.list_stride, w.message_list_stride) * 4 < (1ll << 31);
    const bool narrow_messages =
        narrow_tiles && layers > 1 && narrow_lds_bytes(tg, shape, d.K, tile_message_rows(d.M), tg.tw) <= lds_limit;
    // (layer 0 of a model without message layers keeps the two-phase kernels on rows of more than 32 words)
    const bool half_rows0 = narrow_tiles && !tg.half && (layers > 1 || tg.tw <= 32) &&
                            (g->flags & GTM_GRAPHS_COMPLEMENTARY) && cfg->literals % 2 == 0 &&
                            narrow_lds_bytes(tg, shape, d.K, hv + g->number_of_node_types + 1, tg.tw) <= lds_limit &&
                            !tune(T_NO_HALF_ROWS);
    // words from row to row in LDS (128 bytes apart where that fits; GTM_NARROW_ROWS_AS_STORED, tuning aid: as in memory)
    const bool as_stored = tune(T_NARROW_ROWS_AS_STORED) != nullptr;
    const int row_words0 = half_rows0 && !as_stored
                               ? narrow_row_words(tg, shape, d.K, hv + g->number_of_node_types + 1, lds_limit) : tg.tw;
    const int row_words_m = narrow_messages && !as_stored
                                ? narrow_row_words(tg, shape, d.K, tile_message_rows(d.M), lds_limit) : tg.tw;
    // compiled clause: 8 words of packed 16-bit row entries (16 words of byte offsets on half tiles) + the include words
    const int stride0 = half_rows0 ? w.list_stride : tg.half ? 16 + d.LA + HALF_RECORD_EXTRA_WORDS : two_phase ? 8 + d.LA : w.list_stride;
    SegmentPlan plan{};
    if (half_rows0)
        // rows as k_tile_layer_narrow<ROWS_HALF> stages them: positive literals, node types, all ones
        hipLaunchKernelGGL(k_compile_clauses, dim3(blocks_for(d.C, TPB / 64)), dim3(TPB), 0, st, s->ta_state, d.C,
                           d.LA, d.B, d.filter, cfg->literals, hv, g->number_of_node_types, hv, hv + g->number_of_node_types,
                           row_words0, w.list_stride, order, w.lists, d.K, layers == 1 ? s->clause_weights : nullptr, w.wt);
    else if (tg.half) {
        if (layers == 1 && !tr) {  // one launch over every tile of the range: its tiles may be shared out among the CUs
            TileLayerArgs range{};
            range.tg = tg, range.C = d.C, range.K = d.K, range.tile0 = first / tg.gpt, range.first_graph = first;
            range.n_graphs = n_graphs, range.class_sum = class_sum;
            plan = plan_segments(range, (first + n_graphs - 1) / tg.gpt - range.tile0 + 1, w.segments);
        }
        hipLaunchKernelGGL(k_compile_clauses_half, dim3(blocks_for(d.C, TPB / 64)), dim3(TPB), 0, st,
                           s->ta_state, d.C, d.LA, d.B, d.filter, cfg->literals, g->number_of_node_types, tg.tw, order, w.lists,
                           stride0, d.K, layers == 1 ? s->clause_weights : nullptr, w.wt, plan);
    }
    else if (two_phase)
        hipLaunchKernelGGL(k_compile_clauses_two_phase, dim3(blocks_for(d.C, TPB / 64)), dim3(TPB), 0, st, s->ta_state,
                           d.C, d.LA, d.B, d.filter, cfg->literals, g->number_of_node_types, cfg->literals,
                           tg.rows - 1, tg.tw, order, w.lists, stride0, d.K,
                           layers == 1 ? s->clause_weights : nullptr, w.wt);
    else
        hipLaunchKernelGGL(k_compile_clauses, dim3(blocks_for(d.C, TPB / 64)), dim3(TPB), 0, st, s->ta_state, d.C,
                           d.LA, d.B, d.filter, cfg->literals, 0, g->number_of_node_types, cfg->literals, tg.rows - 1,
                           tg.tw, w.list_stride, order, w.lists, d.K, layers == 1 ? s->clause_weights : nullptr, w.wt);
    if (int rc = check_launch("compile_clauses")) return rc;
    if (layers > 1) {
        hipLaunchKernelGGL(k_fill_i32, dim3(1), dim3(TPB), 0, st, (int32_t *)w.longest_list, (int64_t)(layers - 1), 0);
        if (int rc = check_launch("fill")) return rc;
    }
    for (int l = 1; l < layers; ++l) {
        hipLaunchKernelGGL(k_compile_clauses, dim3(blocks_for(d.C, TPB / 64)), dim3(TPB), 0, st,
                           s->message_ta_state[l - 1], d.C, d.MC, d.B, d.mfilter, 2 * d.M, d.M, 0, 0, d.M, row_words_m,
                           w.message_list_stride, (const uint32_t *)nullptr,
                           w.message_lists + (size_t)(l - 1) * d.C * w.message_list_stride, d.K,
                           l == layers - 1 ? s->clause_weights : nullptr, w.wt, w.longest_list + (l - 1));
        if (int rc = check_launch("compile_clauses")) return rc;
    }
    // layer 0 on narrow tiles takes its clauses by length (GTM_NARROW_IN_ORDER, tuning and test aid: by number)
    const bool by_length = half_rows0 && d.C <= NARROW_ORDER_MAX_CLAUSES && !tune(T_NARROW_IN_ORDER);
    if (by_length) {
        uint32_t *keys = w.stream_order + (size_t)d.C + 2 * NARROW_MAX_STREAMS;
        hipLaunchKernelGGL(k_narrow_order_keys, dim3(blocks_for(d.C, NARROW_ORDER_BLOCK)), dim3(NARROW_ORDER_BLOCK), 0, st,
                           w.lists, w.list_stride, w.message_lists, w.message_list_stride, narrow_messages ? layers - 1 : 0,
                           d.C, shape.streams(), narrow_alive_stride(d.C, shape.streams()), keys, w.stream_order);
        if (int rc = check_launch("narrow_order_keys")) return rc;
        hipLaunchKernelGGL(k_narrow_order_ranks, dim3(blocks_for(d.C, NARROW_ORDER_BLOCK / 64)), dim3(NARROW_ORDER_BLOCK), 0,
                           st, keys, d.C, shape.streams(), narrow_alive_stride(d.C, shape.streams()), w.stream_order);
        if (int rc = check_launch("narrow_order_ranks")) return rc;
    }
    TileLayerArgs a{};
    a.tiles = g->tiles;
    a.tg = tg;
    a.C = d.C;
    a.K = d.K;
    a.wt = w.wt;
    a.bitmap = w.tile_bitmap;
    a.M = d.M;
    a.G = g->number_of_graphs;
    a.node_index = g->node_index;
    a.n_nodes = g->number_of_graph_nodes;
    a.X = g->X;
    a.xpos = tg.half ? g->tiles + tiles_xpos_offset_words(tg, cfg->literals) : nullptr;
    a.walk_factor = 2;
    if (const char *e = tune(T_WIDE_WALK_FACTOR)) a.walk_factor = std::max(1, atoi(e));  // (tuning aid)
    NarrowArgs px{};
    px.alive_stride = narrow_tiles ? narrow_alive_stride(d.C, shape.streams()) : 0;
    px.hv = hv;
    px.n_types = g->number_of_node_types;
    const uint32_t *alive_now = nullptr;  // what the last layer on narrow tiles left for the next one
    auto layer0 = [&](int n_tiles, bool last) {
        a.lists = w.lists;
        a.stride = stride0;
        if (half_rows0) {
            px.alive_in = by_length ? w.stream_order : nullptr;
            px.alive_in_shared = 1;
            px.alive_out = !last && narrow_messages ? w.alive[0] : nullptr;
            px.row_words = row_words0;
            alive_now = px.alive_out;
            return launch_narrow(a, px, shape, n_tiles, ROWS_HALF, last, st);
        }
        alive_now = nullptr;
        if (tg.half) return launch_two_phase_half(a, n_tiles, d.LA / 4, last, &plan, st);
        if (narrow) return launch_two_phase(a, n_tiles, d.LA / 4, last, st);
        if (wide) return launch_two_phase_wide(a, n_tiles, d.LA, tg.stage0 != 0, last, st);
        return launch_tile_layer(a, n_tiles, tg.stage0 ? ROWS_STAGED : ROWS_GLOBAL, last, st);
    };
    if (layers == 1 && !tr) {
        // no truth rows are kept: every tile of the range in one launch
        a.tile0 = first / tg.gpt;
        a.first_graph = first;
        a.n_graphs = n_graphs;
        a.class_sum = class_sum;
        int n_tiles = (first + n_graphs - 1) / tg.gpt - a.tile0 + 1;
        return layer0(n_tiles, true);
    }
    if (layers > 1 && g->total_edges > 0 && (!g->number_of_graph_node_edges || !g->edge || !g->edge_index))
        return fail(GTM_ERR_INVALID, "graphs with edges need number_of_graph_node_edges, edge and edge_index");
    const int tiles_per_launch = tiles_per_batch(tg, batch);
    const int tile_first = first / tg.gpt, tile_last = (first + n_graphs - 1) / tg.gpt;
    const int MW = (d.M + 31) / 32;
    int group = 16;  // words of a truth row per k_tile_node_messages block: its vectors must fit in 64 KB of LDS
    while (group > 1 && ((size_t)32 * group * (MW | 1) + group) * 4 > 64 * 1024) group >>= 1;
    a.message_rows = w.message_rows;
    const size_t fused_lds = tg.slot_words > 0 ? tile_fused_messages_lds_bytes(tg, MW) : 0;
    bool fused_messages = layers > 1 && tg.slot_words > 0 && d.M % 32 == 0 && fused_lds <= 150 * 1024 &&
                          !tune(T_NO_FUSED_MESSAGES);
    if (fused_messages) {
        static thread_local size_t fused_lds_set = 48 * 1024;
        if (fused_lds > fused_lds_set) {
            if (hipFuncSetAttribute((const void *)k_tile_messages_fused, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)fused_lds) != hipSuccess) {
                (void)hipGetLastError();
                fused_messages = false;
            } else {
                fused_lds_set = fused_lds;
            }
        }
    }
    // One tile per workgroup with the vectors in LDS (score_messages.h) where a graph's two sets of vectors are too
    // big for the kernel above.  GTM_MESSAGES_IN_LDS (tuning and test aid): 0 keeps the three launches, 1 prefers
    // this kernel wherever the shape allows it.
    TileMessagesPlan in_lds{};
    {
        const char *e = tune(T_MESSAGES_IN_LDS);
        const bool off = e && atoi(e) == 0, preferred = e && atoi(e) != 0;
        if (layers > 1 && !off && d.C < (1 << 24) && (preferred || !fused_messages)) in_lds = tile_messages_lds_plan(tg, d.M, lds_limit);
    }
    if (in_lds.ok) {
        static thread_local size_t in_lds_set = 48 * 1024;
        if (in_lds.lds_bytes > in_lds_set) {
            // (both forms of the kernel, so that the limit that is remembered holds for either)
            if (hipFuncSetAttribute((const void *)k_tile_messages_in_lds<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)in_lds.lds_bytes) != hipSuccess ||
                hipFuncSetAttribute((const void *)k_tile_messages_in_lds<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)in_lds.lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                in_lds.ok = 0;
            } else {
                in_lds_set = in_lds.lds_bytes;
            }
        }
    }
    if (in_lds.ok) fused_messages = false;
    const bool by_bit = !tune(T_NODE_MESSAGES_BY_ATOMICS);  // tuning aid: the earlier kernel
    if (layers > 1 && !in_lds.ok && (fused_messages || by_bit)) {
        // the clauses of every message bit, for the kernels that build what the nodes send
        hipLaunchKernelGGL(k_message_bit_index, dim3(1), dim3(BIT_INDEX_BLOCK), 0, st, s->hypervectors, d.C, d.MB, d.M,
                           w.bit_start, w.bit_cursor, w.bit_clauses);
        if (int rc = check_launch("message_bit_index")) return rc;
    }
    static thread_local bool node_messages_lds_raised = false;
    if (layers > 1 && !node_messages_lds_raised) {
        hipError_t e = hipFuncSetAttribute((const void *)k_tile_node_messages,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit: %s", hipGetErrorString(e));
        node_messages_lds_raised = true;
    }
    // the clause evaluation of message layer l on the rows just built (a.lists, a.stride, a.longest_list are set)
    auto message_layer = [&](int n_tiles, int l) {
        const bool last = l == layers - 1 && !tr;
        if (!narrow_messages) return launch_tile_layer(a, n_tiles, ROWS_MESSAGES, last, st);
        px.alive_in = alive_now;
        px.alive_in_shared = 0;
        px.row_words = row_words_m;
        px.alive_out = last || l == layers - 1 ? nullptr : w.alive[alive_now == w.alive[0] ? 1 : 0];
        alive_now = px.alive_out;
        return launch_narrow(a, px, shape, n_tiles, ROWS_MESSAGES, last, st);
    };
    for (int t0 = tile_first; t0 <= tile_last; t0 += tiles_per_launch) {
        const int n_tiles = tile_last - t0 + 1 < tiles_per_launch ? tile_last - t0 + 1 : tiles_per_launch;
        a.tile0 = t0;
        a.first_graph = first;
        a.n_graphs = n_graphs;
        a.class_sum = class_sum;
        if (int rc = layer0(n_tiles, false)) return rc;
        for (int l = 1; l < layers; ++l) {
            // the layer's message rows for these tiles (score_tiles.h): one graph per workgroup with its
            // vectors in LDS when they fit, else three launches with the vectors in global memory
            if (in_lds.ok) {
                profile_start("k_tile_messages_in_lds", st);
                hipLaunchKernelGGL(tg.tw > 32 ? k_tile_messages_in_lds<true> : k_tile_messages_in_lds<false>, dim3(n_tiles),
                                   dim3(TILE_MESSAGES_LDS_BLOCK), in_lds.lds_bytes, st,
                                   w.tile_bitmap, d.C, tg, t0, g->number_of_graphs, d.M, s->hypervectors, d.MB, alive_now,
                                   narrow_tiles ? shape.streams() : TILE_MESSAGES_LDS_BLOCK / 16, px.alive_stride, g->node_index, g->number_of_graph_nodes, g->number_of_graph_node_edges,
                                   g->edge_index, g->edge, g->total_edges > 0 ? 1 : 0, in_lds.main_words, in_lds.range_words,
                                   w.message_rows);
                if (int rc = check_launch("tile_messages_in_lds")) return rc;
                profile_stop(st);
                a.lists = w.message_lists + (size_t)(l - 1) * d.C * w.message_list_stride;
                a.stride = w.message_list_stride;
                a.longest_list = w.longest_list + (l - 1);
                if (int rc = message_layer(n_tiles, l)) return rc;
                continue;
            }
            if (fused_messages) {
                profile_start("k_tile_messages_fused", st);
                hipLaunchKernelGGL(k_tile_messages_fused, dim3(tg.gpt, n_tiles), dim3(TILE_FUSED_MESSAGES_BLOCK),
                                   fused_lds, st, w.tile_bitmap, d.C, tg, t0, g->number_of_graphs, d.M, MW, w.bit_start,
                                   w.bit_clauses, g->node_index, g->number_of_graph_nodes, g->number_of_graph_node_edges,
                                   g->edge_index, g->edge, g->total_edges > 0 ? 1 : 0, w.message_rows);
                if (int rc = check_launch("tile_messages_fused")) return rc;
                profile_stop(st);
                a.lists = w.message_lists + (size_t)(l - 1) * d.C * w.message_list_stride;
                a.stride = w.message_list_stride;
                a.longest_list = w.longest_list + (l - 1);
                if (int rc = message_layer(n_tiles, l)) return rc;
                continue;
            }
            profile_start("k_tile_node_messages + k_tile_edge_messages + k_tile_pack_messages", st);
            if (by_bit) {
                const int pack = tg.tw <= 32 && !tune(T_NO_TILE_PACK) ? 64 / tg.tw : 1;  // narrow tiles share a wave
                const int blocks_per_group = (MW + NODE_MESSAGES_BY_BIT_WAVES - 1) / NODE_MESSAGES_BY_BIT_WAVES;
                const int n_groups = (n_tiles + pack - 1) / pack;
                hipLaunchKernelGGL(k_tile_node_messages_by_bit, dim3((unsigned)((n_groups + 7) / 8 * 8 * blocks_per_group)),
                                   dim3(64 * NODE_MESSAGES_BY_BIT_WAVES), 0, st, w.tile_bitmap, d.C, tg.tw, w.bit_start,
                                   w.bit_clauses, d.M, MW, n_tiles, pack, blocks_per_group, n_groups, w.sent);
            }
            else
            hipLaunchKernelGGL(k_tile_node_messages, dim3((tg.tw + group - 1) / group, n_tiles),
                               dim3(TILE_MESSAGES_BLOCK), ((size_t)32 * group * (MW | 1) + group) * 4, st, w.tile_bitmap, d.C, tg.tw,
                               group, s->hypervectors, d.MB, MW, w.sent);
            if (int rc = check_launch("tile_node_messages")) return rc;
            const int64_t vector_words = (int64_t)n_tiles * tg.tw * 32 * MW;
            hipLaunchKernelGGL(k_fill_i32, dim3(blocks_for(vector_words, TPB)), dim3(TPB), 0, st, (int32_t *)w.got,
                               vector_words, 0);
            if (int rc = check_launch("fill")) return rc;
            if (g->total_edges > 0) {
                hipLaunchKernelGGL(k_tile_edge_messages, dim3(blocks_for(vector_words, TPB)), dim3(TPB), 0, st, w.sent, tg,
                                   t0, g->number_of_graphs, d.M, MW, g->node_index, g->number_of_graph_nodes,
                                   g->number_of_graph_node_edges, g->edge_index, g->edge, vector_words, w.got);
                if (int rc = check_launch("tile_edge_messages")) return rc;
            }
            hipLaunchKernelGGL(k_tile_pack_messages, dim3((unsigned)((n_tiles + 7) / 8 * 8 * ((tg.tw + 1) / 2))), dim3(256),
                               (size_t)64 * (MW + 1) * 4, st, w.got, tg, t0, g->number_of_graphs, d.M, MW,
                               g->number_of_graph_nodes, w.message_rows, (tg.tw + 1) / 2, n_tiles);
            if (int rc = check_launch("tile_pack_messages")) return rc;
            profile_stop(st);
            a.lists = w.message_lists + (size_t)(l - 1) * d.C * w.message_list_stride;
            a.stride = w.message_list_stride;
            a.longest_list = w.longest_list + (l - 1);
            if (int rc = message_layer(n_tiles, l)) return rc;
        }
        if (tr) {
            const int g_lo = std::max(first, t0 * tg.gpt), g_hi = std::min(first + n_graphs, (t0 + n_tiles) * tg.gpt);
            if (g_hi > g_lo) {
                profile_start("k_tile_transform", st);
                hipLaunchKernelGGL(k_tile_transform, dim3(g_hi - g_lo), dim3(TILE_TRANSFORM_BLOCK),
                                   ((size_t)(d.C + 31) / 32 + TILE_TRANSFORM_BLOCK / 64) * 4, st, w.tile_bitmap, tg, t0, g_lo, first,
                                   d.C, d.K, g->number_of_graph_nodes, s->clause_weights, tr->transformed, tr->nodewise, tr->width,
                                   class_sum);
                if (int rc = check_launch("tile_transform")) return rc;
                profile_stop(st);
            }
        }
    }
    return GTM_OK;
}

// The tile path of gtm_score / gtm_transform needs a data set with tiles of a usable geometry.
// GTM_NO_TILE_TRANSFORM (tuning aid) keeps gtm_transform on the dense path.
bool tiles_usable(const gtm_config *cfg, const gtm_graphs *graphs, int classes, TileGeom *tg) {
    if (!graphs || !graphs->tiles || graphs->number_of_graphs < 1 || graphs->number_of_node_types < 1) return false;
    *tg = geometry_for(cfg, graphs, classes);
    // with message layers a 64-slot block of message vectors has to fit in 64 KB of LDS
    if (cfg->depth > 1 && (size_t)64 * ((cfg->message_size + 31) / 32 + 1) * 4 > 64 * 1024) return false;
    return tg->ok != 0;
}

bool transform_uses_tiles(const gtm_config *cfg, const gtm_graphs *graphs, int classes, TileGeom *tg) {
    return !tune(T_NO_TILE_TRANSFORM) && tiles_usable(cfg, graphs, classes, tg);
}

}  // namespace

// =============================================================== C ABI

extern "C" {

int gtm_abi_version(void) { return GTM_ABI_VERSION; }

const char *gtm_last_error(void) { return g_error; }

int gtm_prepare(const gtm_config *cfg, uint64_t step, uint32_t *ta_state, int32_t *clause_weights, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (!ta_state || !clause_weights) return fail(GTM_ERR_INVALID, "NULL buffer");
    hipStream_t st = (hipStream_t)stream;
    int64_t words = (int64_t)d.C * d.LA * d.B;
    hipLaunchKernelGGL(k_prepare_bank, dim3(blocks_for(words, TPB)), dim3(TPB), 0, st, ta_state, words, d.B);
    if (int rc = check_launch("prepare_bank")) return rc;
    Key k = key_of(cfg);
    hipLaunchKernelGGL(k_prepare_weights, dim3(blocks_for((int64_t)d.K * d.C, TPB)), dim3(TPB), 0, st, clause_weights,
                       d.K, d.C, cfg->negative_clauses, k.k0, k.k1, (uint32_t)step);
    return check_launch("prepare_weights");
}

int gtm_prepare_message_ta_state(const gtm_config *cfg, uint32_t *message_ta_state, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (!message_ta_state) return fail(GTM_ERR_INVALID, "NULL buffer");
    int64_t words = (int64_t)d.C * d.MC * d.B;
    hipLaunchKernelGGL(k_prepare_bank, dim3(blocks_for(words, TPB)), dim3(TPB), 0, (hipStream_t)stream,
                       message_ta_state, words, d.B);
    return check_launch("prepare_bank");
}

int gtm_calculate_messages(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph, int32_t n_graphs,
                           const uint32_t *ta_state, uint32_t *include_plane, uint32_t *clause_node_output,
                           int32_t *number_of_include_actions, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_graph, n_graphs)) return rc;
    if (!ta_state || !clause_node_output || !include_plane) return fail(GTM_ERR_INVALID, "NULL buffer");
    hipStream_t st = (hipStream_t)stream;
    if (int rc = op_include_plane(d, ta_state, d.LA, d.filter, include_plane, number_of_include_actions, 0, st)) return rc;
    return launch_clause_node_bits(d, graphs, first_graph, n_graphs, include_plane, d.LA, graphs->X, 0, cfg->max_nodes,
                                   nullptr, clause_node_output, st);
}

int gtm_exchange_messages(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph, int32_t n_graphs,
                          const uint32_t *hypervectors, const uint32_t *clause_node_output, uint32_t *clause_X,
                          void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_graph, n_graphs)) return rc;
    if (!hypervectors || !clause_node_output || !clause_X) return fail(GTM_ERR_INVALID, "NULL buffer");
    return op_exchange(d, cfg, graphs, first_graph, n_graphs, hypervectors, clause_node_output, clause_X,
                       (hipStream_t)stream);
}

int gtm_calculate_messages_conditional(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph,
                                       int32_t n_graphs, const uint32_t *message_ta_state, uint32_t *include_plane,
                                       const uint32_t *clause_node_output_condition, uint32_t *clause_node_output,
                                       int32_t *number_of_include_actions, const uint32_t *clause_X, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_graph, n_graphs)) return rc;
    if (!message_ta_state || !clause_node_output_condition || !clause_node_output || !clause_X || !include_plane)
        return fail(GTM_ERR_INVALID, "NULL buffer");
    hipStream_t st = (hipStream_t)stream;
    if (int rc = op_include_plane(d, message_ta_state, d.MC, d.mfilter, include_plane, number_of_include_actions, 1, st))
        return rc;
    return launch_clause_node_bits(d, graphs, first_graph, n_graphs, include_plane, d.MC, clause_X, 1, cfg->max_nodes,
                                   clause_node_output_condition, clause_node_output, st);
}

int gtm_evaluate(const gtm_config *cfg, const gtm_graphs *graphs, int32_t first_graph, int32_t n_graphs,
                 const uint32_t *clause_node_output, const int32_t *clause_weights, int32_t *class_sum,
                 void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_graph, n_graphs)) return rc;
    if (!clause_node_output || !clause_weights || !class_sum) return fail(GTM_ERR_INVALID, "NULL buffer");
    return op_class_sums(d, graphs, first_graph, n_graphs, clause_node_output, clause_weights, class_sum,
                         (hipStream_t)stream);
}

}  // extern "C"

namespace {

// Training operators take the example's node count from the host copy that
// the caller passes (the driver loop reads it once per dataset).
int op_select_clause_node(const Dims &d, const gtm_config *cfg, int n_nodes, uint64_t step, const uint32_t *bitmap,
                          int32_t *clause_node, hipStream_t st) {
    Key k = key_of(cfg);
    hipLaunchKernelGGL(k_select_clause_node, dim3(blocks_for(d.C, TPB)), dim3(TPB), 0, st, bitmap, d.C, d.NC, n_nodes,
                       k.k0, k.k1, (uint32_t)step, clause_node);
    return check_launch("select_clause_node");
}

int op_select_clause_updates(const Dims &d, const gtm_config *cfg, uint64_t step, int32_t *weights,
                             const int32_t *class_sum, const int32_t *y_row, const int32_t *clause_node,
                             int32_t *update, hipStream_t st) {
    Key k = key_of(cfg);
    hipLaunchKernelGGL(k_select_clause_updates, dim3(blocks_for(d.C, TPB)), dim3(TPB), 0, st, weights, class_sum, y_row,
                       d.K, d.C, cfg->threshold, cfg->negative_clauses, q_threshold(cfg->q, cfg->classes), k.k0, k.k1,
                       (uint32_t)step, clause_node, update);
    return check_launch("select_clause_updates");
}

int op_update(const Dims &d, const gtm_config *cfg, uint64_t step, int bank_id, uint32_t *bank, int chunks,
              const int32_t *clause_node, const int32_t *n_incl, const uint32_t *rows, const int32_t *update,
              hipStream_t st) {
    Key k = key_of(cfg);
    int64_t items = (int64_t)d.C * chunks;
    hipLaunchKernelGGL(k_update, dim3(blocks_for(items, TPB)), dim3(TPB), 0, st, bank, d.C, chunks, d.B, d.K,
                       cfg->boost_true_positive_feedback, cfg->max_included_literals,
                       feedback_threshold(cfg->s[bank_id]), k.k0, k.k1, (uint32_t)step, (uint32_t)bank_id, clause_node,
                       n_incl, rows, update);
    return check_launch("update");
}

}  // namespace

extern "C" {

int gtm_select_clause_node(const gtm_config *cfg, const gtm_graphs *graphs, int32_t example, uint64_t step,
                           const uint32_t *clause_node_output, int32_t *clause_node, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, example, 1)) return rc;
    if (!clause_node_output || !clause_node) return fail(GTM_ERR_INVALID, "NULL buffer");
    uint32_t n = 0;
    hipError_t e = hipMemcpyAsync(&n, graphs->number_of_graph_nodes + example, 4, hipMemcpyDeviceToHost,
                                  (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "reading node count: %s", hipGetErrorString(e));
    return op_select_clause_node(d, cfg, (int)n, step, clause_node_output, clause_node, (hipStream_t)stream);
}

int gtm_select_clause_updates(const gtm_config *cfg, uint64_t step, int32_t *clause_weights,
                              const int32_t *class_sum, const int32_t *encoded_Y, int32_t example,
                              const int32_t *clause_node, int32_t *class_clause_update, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (!clause_weights || !class_sum || !encoded_Y || !clause_node || !class_clause_update || example < 0)
        return fail(GTM_ERR_INVALID, "NULL buffer or negative example");
    return op_select_clause_updates(d, cfg, step, clause_weights, class_sum, encoded_Y + (int64_t)example * d.K,
                                    clause_node, class_clause_update, (hipStream_t)stream);
}

int gtm_update(const gtm_config *cfg, const gtm_graphs *graphs, int32_t example, uint64_t step,
               uint32_t *ta_state, const int32_t *clause_node, const int32_t *number_of_include_actions,
               const int32_t *class_clause_update, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, example, 1)) return rc;
    if (!ta_state || !clause_node || !number_of_include_actions || !class_clause_update)
        return fail(GTM_ERR_INVALID, "NULL buffer");
    uint32_t base = 0;
    hipError_t e = hipMemcpyAsync(&base, graphs->node_index + example, 4, hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "reading node index: %s", hipGetErrorString(e));
    return op_update(d, cfg, step, 0, ta_state, d.LA, clause_node, number_of_include_actions,
                     graphs->X + (int64_t)base * d.LA, class_clause_update, (hipStream_t)stream);
}

int gtm_update_message(const gtm_config *cfg, uint64_t step, int32_t bank, uint32_t *message_ta_state,
                       const int32_t *clause_node, const int32_t *number_of_include_actions,
                       const uint32_t *clause_X, const int32_t *class_clause_update, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (bank < 1 || bank >= cfg->depth) return fail(GTM_ERR_INVALID, "bank=%d outside 1..%d", bank, cfg->depth - 1);
    if (!message_ta_state || !clause_node || !number_of_include_actions || !clause_X || !class_clause_update)
        return fail(GTM_ERR_INVALID, "NULL buffer");
    return op_update(d, cfg, step, bank, message_ta_state, d.MC, clause_node, number_of_include_actions, clause_X,
                     class_clause_update, (hipStream_t)stream);
}

static int read_bank(const gtm_config *cfg, const uint32_t *bank, int32_t chunks, int32_t literals, int actions,
                     uint32_t *out, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (!bank || !out) return fail(GTM_ERR_INVALID, "NULL buffer");
    if (chunks < 1 || literals < 1 || literals > chunks * 32)
        return fail(GTM_ERR_INVALID, "chunks=%d literals=%d", chunks, literals);
    int64_t total = (int64_t)d.C * literals;
    hipLaunchKernelGGL(k_read_bank, dim3(blocks_for(total, TPB)), dim3(TPB), 0, (hipStream_t)stream, bank, d.C, chunks,
                       d.B, literals, actions, out);
    return check_launch("read_bank");
}

int gtm_get_ta_states(const gtm_config *cfg, const uint32_t *bank, int32_t chunks, int32_t literals, uint32_t *out,
                      void *stream) {
    return read_bank(cfg, bank, chunks, literals, 0, out, stream);
}

int gtm_get_hyperliterals(const gtm_config *cfg, const uint32_t *bank, int32_t chunks, int32_t literals,
                          uint32_t *out, void *stream) {
    return read_bank(cfg, bank, chunks, literals, 1, out, stream);
}

size_t gtm_transform_workspace_bytes(const gtm_config *cfg, const gtm_graphs *graphs, int32_t batch) {
    Dims d;
    if (validate(cfg, &d) || batch < 1) return 0;
    TileGeom tg;
    const bool tiles = transform_uses_tiles(cfg, graphs, d.K, &tg);
    return carve_score(d, cfg, batch, nullptr, tiles ? &tg : nullptr, true).bytes;
}

int gtm_transform(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, int32_t first_graph,
                  int32_t n_graphs, int32_t batch, void *workspace, size_t workspace_bytes, int32_t *transformed,
                  int32_t *nodewise, int32_t width, int32_t *class_sum, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_graph, n_graphs)) return rc;
    if (int rc = validate_state(cfg, state)) return rc;
    if (batch < 1) return fail(GTM_ERR_INVALID, "batch=%d", batch);
    if (!transformed || !class_sum) return fail(GTM_ERR_INVALID, "NULL output");
    if (nodewise && (width < 1 || width > cfg->max_nodes))
        return fail(GTM_ERR_INVALID, "width=%d outside [1, max_nodes=%d]", width, cfg->max_nodes);
    TileGeom tg;
    const bool tiles = transform_uses_tiles(cfg, graphs, d.K, &tg);
    ScoreWs w = carve_score(d, cfg, batch, (char *)workspace, tiles ? &tg : nullptr, true);
    if (!workspace || workspace_bytes < w.bytes)
        return fail(GTM_ERR_INVALID, "workspace of %zu bytes needed, %zu given", w.bytes, workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    if (n_graphs == 0) return GTM_OK;
    if (tiles) {
        // the truth rows that the tile kernels of gtm_score compute, kept for the last layer too
        if (int rc = check_tiles(tg, cfg, graphs)) return rc;
        const TransformOut out{transformed, nodewise, width};
        return score_on_tiles(d, cfg, graphs, state, tg, w, first_graph, n_graphs, batch, class_sum, st, &out);
    }
    for (int done = 0; done < n_graphs; done += batch) {
        int nb = n_graphs - done < batch ? n_graphs - done : batch;
        uint32_t *final_bitmap = nullptr;
        uint32_t *layers[1] = {w.clause_X};
        if (int rc = run_evaluate(d, cfg, graphs, state, first_graph + done, nb, w.inc_t, w.bitmap_a, w.bitmap_b, layers,
                                  false, nullptr, class_sum + (int64_t)done * d.K, &final_bitmap, st))
            return rc;
        int64_t total = (int64_t)nb * d.C;
        hipLaunchKernelGGL(k_transform, dim3(blocks_for(total, TPB)), dim3(TPB), 0, st, final_bitmap, d.C, d.NC,
                           graphs->number_of_graph_nodes, first_graph + done, total, transformed + (int64_t)done * d.C);
        if (int rc = check_launch("transform")) return rc;
        if (nodewise) {
            int64_t cells = total * width;
            hipLaunchKernelGGL(k_transform_nodewise, dim3(blocks_for(cells, TPB)), dim3(TPB), 0, st, final_bitmap, d.C,
                               d.NC, width, graphs->number_of_graph_nodes, first_graph + done, cells,
                               nodewise + (int64_t)done * d.C * width);
            if (int rc = check_launch("transform_nodewise")) return rc;
        }
    }
    return GTM_OK;
}

int gtm_tuning_set(const char *name, const char *value) {
    if (!name) return fail(GTM_ERR_INVALID, "name is NULL");
    for (int i = 0; i < T_COUNT; ++i)
        if (strcmp(name, g_switch_name[i]) == 0) {
            if (value && strlen(value) >= sizeof g_switches.value[i])
                return fail(GTM_ERR_INVALID, "value of %s longer than %zu characters", name, sizeof g_switches.value[i] - 1);
            g_switches.put(i, value);
            return GTM_OK;
        }
    return fail(GTM_ERR_INVALID, "%s is not a switch of this library", name);
}

const char *gtm_tuning_get(const char *name) {
    if (!name) return nullptr;
    for (int i = 0; i < T_COUNT; ++i)
        if (strcmp(name, g_switch_name[i]) == 0) return tune((Switch)i);
    return nullptr;
}

int gtm_tuning_reload(void) {
    g_switches = Switches();
    return GTM_OK;
}

int gtm_profile_enable(int on) {
    g_prof.on = on != 0;
    g_prof.used = 0;
    if (!on) {
        // no HIP object of this library's outlives the measurement (none is left for process exit)
        for (int i = 0; i < g_prof.created; ++i) {
            (void)hipEventDestroy(g_prof.start[i]);
            (void)hipEventDestroy(g_prof.stop[i]);
        }
        g_prof.created = 0;
    }
    return GTM_OK;
}

int gtm_profile_read(const char **kernel_name, int32_t *launches, double *total_ms) {
    if (!kernel_name || !launches || !total_ms) return fail(GTM_ERR_INVALID, "NULL output");
    double total = 0.0;
    for (int i = 0; i < g_prof.used; ++i) {
        hipError_t e = hipEventSynchronize(g_prof.stop[i]);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, g_prof.start[i], g_prof.stop[i]);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "reading profile events: %s", hipGetErrorString(e));
        total += ms;
    }
    *kernel_name = g_prof.name;
    *launches = g_prof.used;
    *total_ms = total;
    g_prof.used = 0;
    return GTM_OK;
}

int gtm_profile_read_kernel(int32_t index, const char **kernel_name, int32_t *launches, double *total_ms) {
    if (!kernel_name || !launches || !total_ms || index < 0) return fail(GTM_ERR_INVALID, "NULL output or negative index");
    *kernel_name = nullptr, *launches = 0, *total_ms = 0.0;
    // the index-th distinct name in the order of first use (names are string literals of this file)
    const char *wanted = nullptr;
    int seen = 0;
    for (int i = 0; i < g_prof.used && !wanted; ++i) {
        bool earlier = false;
        for (int j = 0; j < i && !earlier; ++j) earlier = strcmp(g_prof.name_of[j], g_prof.name_of[i]) == 0;
        if (!earlier && seen++ == index) wanted = g_prof.name_of[i];
    }
    if (!wanted) return GTM_OK;
    double total = 0.0;
    int count = 0;
    for (int i = 0; i < g_prof.used; ++i) {
        if (strcmp(g_prof.name_of[i], wanted) != 0) continue;
        hipError_t e = hipEventSynchronize(g_prof.stop[i]);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, g_prof.start[i], g_prof.stop[i]);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "reading profile events: %s", hipGetErrorString(e));
        total += ms;
        ++count;
    }
    *kernel_name = wanted, *launches = count, *total_ms = total;
    return GTM_OK;
}

int gtm_graphs_properties(const gtm_config *cfg, const gtm_graphs *graphs, uint32_t *properties, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, 0, 0)) return rc;
    if (!properties) return fail(GTM_ERR_INVALID, "properties is NULL");
    if (cfg->literals % 2 != 0) return fail(GTM_ERR_INVALID, "literals=%d is odd", cfg->literals);
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_fill_i32, dim3(1), dim3(TPB), 0, st, (int32_t *)properties, (int64_t)2, 0);
    if (int rc = check_launch("fill")) return rc;
    const int64_t items = graphs->total_nodes > graphs->number_of_graphs ? graphs->total_nodes : graphs->number_of_graphs;
    hipLaunchKernelGGL(k_graphs_properties, dim3(blocks_for(items, TPB)), dim3(TPB), 0, st, graphs->X, graphs->total_nodes,
                       d.LA, cfg->literals, graphs->number_of_graph_nodes, graphs->number_of_graphs, properties);
    return check_launch("graphs_properties");
}

size_t gtm_tiles_bytes(const gtm_config *cfg, const gtm_graphs *graphs) {
    Dims d;
    if (validate(cfg, &d) || !graphs || graphs->number_of_graphs < 1 || graphs->number_of_node_types < 1) return 0;
    TileGeom tg = geometry_for(cfg, graphs, d.K);
    if (!tg.ok) return 0;
    // bit rows, one 64-bit population count per row, the literal order
    if (tg.half) return (tiles_xpos_offset_words(tg, cfg->literals) + tiles_xpos_words(tg, cfg->literals)) * 4;
    return tiles_words(tg) * 4 + (size_t)tg.rows * 8 + (size_t)cfg->literals * 4;
}

int gtm_build_tiles(const gtm_config *cfg, const gtm_graphs *graphs, uint32_t *tiles, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, 0, 0)) return rc;
    if (!tiles) return fail(GTM_ERR_INVALID, "tiles is NULL");
    TileGeom tg = geometry_for(cfg, graphs, d.K);
    if (!tg.ok) return fail(GTM_ERR_INVALID, "this data set's shape has no tile layout (gtm_tiles_bytes() == 0)");
    hipStream_t st = (hipStream_t)stream;
    int64_t total = (int64_t)tg.n_tiles * tg.rows * tg.tw;
    hipLaunchKernelGGL(k_build_tiles, dim3(blocks_for(total, TPB)), dim3(TPB), 0, st, graphs->X, graphs->node_type,
                       graphs->node_index, graphs->number_of_graph_nodes, graphs->number_of_graphs, d.LA,
                       cfg->literals, graphs->number_of_node_types, tg, total, tiles);
    if (int rc = check_launch("build_tiles")) return rc;
    int32_t *counts = (int32_t *)(tiles + tiles_words(tg));
    hipLaunchKernelGGL(k_fill_i32, dim3(blocks_for(tg.rows * 2, TPB)), dim3(TPB), 0, st, counts, (int64_t)tg.rows * 2, 0);
    if (int rc = check_launch("fill")) return rc;
    int64_t total_rows = (int64_t)tg.n_tiles * tg.rows;
    hipLaunchKernelGGL(k_row_counts, dim3(blocks_for(total_rows, TPB)), dim3(TPB), 0, st, tiles, tg, total_rows,
                       (unsigned long long *)counts);
    if (int rc = check_launch("row_counts")) return rc;
    hipLaunchKernelGGL(k_row_order, dim3(blocks_for(cfg->literals, TPB)), dim3(TPB), 0, st,
                       (const unsigned long long *)counts, cfg->literals, (uint32_t *)(counts + (size_t)tg.rows * 2));
    if (int rc = check_launch("row_order")) return rc;
    if (tg.half) {
        const int64_t slots = (int64_t)tg.n_tiles * tg.tw * 32;
        hipLaunchKernelGGL(k_build_xpos, dim3(blocks_for(slots, TPB)), dim3(TPB), 0, st, graphs->X, graphs->node_index,
                           graphs->number_of_graph_nodes, graphs->number_of_graphs, d.LA, tg, slots,
                           tiles + tiles_xpos_offset_words(tg, cfg->literals));
        if (int rc = check_launch("build_xpos")) return rc;
    }
    remember_tiles(tiles, tg, cfg, graphs);
    return GTM_OK;
}

// The tile path runs when the data set carries tiles (gtm_build_tiles) of a supported shape.
static bool score_uses_tiles(const gtm_config *cfg, const gtm_graphs *graphs, int classes, TileGeom *tg) {
    return tiles_usable(cfg, graphs, classes, tg);
}

size_t gtm_score_workspace_bytes(const gtm_config *cfg, const gtm_graphs *graphs, int32_t batch) {
    Dims d;
    if (validate(cfg, &d) || batch < 1) return 0;
    TileGeom tg;
    bool tiles = score_uses_tiles(cfg, graphs, d.K, &tg);
    return carve_score(d, cfg, batch, nullptr, tiles ? &tg : nullptr).bytes;
}

int gtm_score(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, int32_t first_graph,
              int32_t n_graphs, int32_t batch, void *workspace, size_t workspace_bytes, int32_t *class_sum,
              void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_graph, n_graphs)) return rc;
    if (int rc = validate_state(cfg, state)) return rc;
    if (batch < 1) return fail(GTM_ERR_INVALID, "batch=%d", batch);
    if (!class_sum) return fail(GTM_ERR_INVALID, "class_sum is NULL");
    TileGeom tg;
    bool tiles = score_uses_tiles(cfg, graphs, d.K, &tg);
    ScoreWs w = carve_score(d, cfg, batch, (char *)workspace, tiles ? &tg : nullptr);
    if (!workspace || workspace_bytes < w.bytes)
        return fail(GTM_ERR_INVALID, "workspace of %zu bytes needed, %zu given", w.bytes, workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    if (n_graphs == 0) return GTM_OK;
    if (tiles) {
        if (int rc = check_tiles(tg, cfg, graphs)) return rc;
        return score_on_tiles(d, cfg, graphs, state, tg, w, first_graph, n_graphs, batch, class_sum, st);
    }
    for (int done = 0; done < n_graphs; done += batch) {
        int nb = n_graphs - done < batch ? n_graphs - done : batch;
        uint32_t *final_bitmap = nullptr;
        uint32_t *layers[1] = {w.clause_X};
        if (int rc = run_evaluate(d, cfg, graphs, state, first_graph + done, nb, w.inc_t, w.bitmap_a, w.bitmap_b, layers,
                                  false, nullptr, class_sum + (int64_t)done * d.K, &final_bitmap, st))
            return rc;
    }
    return GTM_OK;
}

// ---- gtm_score for callers that cannot allocate -----------------------------------------------
// The workspace of gtm_score lives in a file-scope device array instead of a caller's buffer.
// Every GPU the library runs on holds its own copy of the array, at its own address, until the
// process ends; the address is looked up once per device and only that pointer is ever handed to
// kernels (the array's name is a host-side stand-in, not a device address).
constexpr size_t GTM_STATIC_SCRATCH_BYTES = (size_t)16 << 20;
constexpr int GTM_STATIC_SCRATCH_DEVICES = 64;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[GTM_STATIC_SCRATCH_BYTES];
static void *g_scratch_of_device[GTM_STATIC_SCRATCH_DEVICES];  // filled on a device's first call
static std::mutex g_scratch_mutex;

static int static_scratch(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= GTM_STATIC_SCRATCH_DEVICES) return fail(GTM_ERR_INVALID, "device %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_of_device[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // with `dev` current: that device's copy
        if (e != hipSuccess || !ptr)
            return fail(GTM_ERR_HIP, "address of the static scratch array on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_of_device[dev] = ptr;
    }
    *out = g_scratch_of_device[dev];
    return GTM_OK;
}

size_t gtm_score_static_scratch_bytes(void) { return GTM_STATIC_SCRATCH_BYTES; }

int gtm_score_static(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, int32_t first_graph,
                     int32_t n_graphs, int32_t batch, int32_t *class_sum, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (batch < 1) return fail(GTM_ERR_INVALID, "batch=%d", batch);
    const size_t need = gtm_score_workspace_bytes(cfg, graphs, batch);
    if (need == 0) return fail(GTM_ERR_INVALID, "invalid configuration");
    if (need > GTM_STATIC_SCRATCH_BYTES)
        return fail(GTM_ERR_INVALID,
                    "this model and batch need %zu bytes of scratch; the allocation-free entry point has %zu "
                    "(use a smaller batch, or gtm_score with a workspace of the caller's)",
                    need, GTM_STATIC_SCRATCH_BYTES);
    void *ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    // the launch timing of gtm_profile_enable creates events: not on this path (this thread's calls only;
    // the switch itself, which other threads read, is not touched)
    g_prof_quiet = true;
    const int rc = gtm_score(cfg, graphs, state, first_graph, n_graphs, batch, ptr, GTM_STATIC_SCRATCH_BYTES, class_sum, stream);
    g_prof_quiet = false;
    return rc;
}

}  // extern "C"

namespace {

// How long a device-wide wait of the one-launch training kernels may last: a poll cap that only the
// tests use (GTM_FIT_SPIN_LIMIT = a number of polls, or "abort" = give up at the first wait whatever
// it shows) and 5 seconds of the device's wall clock otherwise.
struct WaitBound {
    uint32_t spin_limit;
    unsigned long long wait_ticks;
    int force_abort;
};
WaitBound wait_bound(int dev) {
    WaitBound b{0xFFFFFFFFu, 0ull, 0};
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0) {
        (void)hipGetLastError();
        khz = 100000;  // 100 MHz
    }
    b.wait_ticks = 5ull * 1000ull * (unsigned long long)khz;
    if (const char *e = tune(T_FIT_SPIN_LIMIT)) {
        b.force_abort = strcmp(e, "abort") == 0;
        if (!b.force_abort) b.spin_limit = (uint32_t)strtoul(e, nullptr, 10);
    }
    return b;
}

// `_fit`'s inner loop as one cooperative launch (fit_persistent.h).  Returns
// GTM_OK with *done = false when this device / shape cannot run it, so that the
// caller falls back to per-example launches.
int fit_persistent(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, const TileGeom &tg,
                   const FitWs &w, const int32_t *encoded_Y, int first_example, int n_examples, uint64_t first_step,
                   hipStream_t st, bool *done) {
    *done = false;
    if (tune(T_NO_PERSISTENT_FIT) || d.K > FITP_BLOCK) return GTM_OK;
    int dev = 0, coop = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return GTM_OK;
    if (hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev) != hipSuccess || !coop) return GTM_OK;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return GTM_OK;

    FitPersistParams p{};
    p.max_words = tg.slot_words > 0 ? tg.slot_words : 1;
    // graphs of one or two nodes: the nodes are tested on their own literal words, no rows are staged
    p.direct = g->max_number_of_graph_nodes <= FITP_DIRECT_NODES && !tune(T_NO_DIRECT_FIT);
    p.node_type = g->node_type;
    p.rows_words = p.direct ? 0 : (cfg->literals + g->number_of_node_types + 1) * p.max_words;
    p.x_words = (g->max_number_of_graph_nodes > 0 ? g->max_number_of_graph_nodes : 1) * d.LA;
    p.order = g->tiles + tiles_words(tg) + (size_t)tg.rows * 2;
    // One clause per wave and step. Few clauses per group keep a step's feedback short, few groups
    // keep the exchange of the class sums short: the clauses are spread over all CUs (8 to 12 per
    // group measured best on 2,000 and 2,500 clauses), but a group gets at least 8 where their
    // automata fit in LDS.
    auto lds_bytes = [&](int per_group) {
        return (2 * (size_t)p.rows_words + (size_t)per_group * d.LA * d.B + 2 * (size_t)per_group +
                2 * (size_t)d.K + 5 * (size_t)per_group * d.K + (size_t)per_group * d.LA * d.K + 2 * (size_t)p.x_words +
                (size_t)cfg->literals + 8 * (size_t)d.K) * 4;
    };
    const size_t lds_limit = 150 * 1024;
    int per_group = (d.C + cus - 1) / cus;
    const int preferred = 8;
    if (per_group < preferred && lds_bytes(preferred) <= lds_limit) per_group = preferred;
    if (const char *e = tune(T_FIT_PER_GROUP)) {  // tuning: clauses per group, at least C / CUs
        const int asked = atoi(e);
        if (asked >= (d.C + cus - 1) / cus && asked <= FITP_BLOCK) per_group = asked;
    }
    if (lds_bytes(per_group) > lds_limit) return GTM_OK;
    const int groups = (d.C + per_group - 1) / per_group;
    p.clauses_per_group = per_group;
    const size_t lds = lds_bytes(per_group);
    // one instance per width of the automata in registers (the widest would cost the others registers)
    const int variant = d.B <= 8 ? 0 : d.B <= 16 ? 1 : 2;
    const void *kernel = variant == 0   ? (const void *)k_fit_persistent<8>
                         : variant == 1 ? (const void *)k_fit_persistent<16>
                                        : (const void *)k_fit_persistent<32>;
    static thread_local size_t lds_set_of[3] = {48 * 1024, 48 * 1024, 48 * 1024};
    size_t &lds_set = lds_set_of[variant];
    if (lds > lds_set) {
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GTM_OK;
        }
        lds_set = lds;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, FITP_BLOCK, lds) != hipSuccess ||
        per_cu < 1 || groups > per_cu * cus) {
        (void)hipGetLastError();
        return GTM_OK;
    }

    Key key = key_of(cfg);
    p.tiles = g->tiles;
    p.X = g->X;
    p.node_index = g->node_index;
    p.n_nodes = g->number_of_graph_nodes;
    p.encoded_Y = encoded_Y;
    p.tg = tg;
    p.first_example = first_example;
    p.n_examples = n_examples;
    p.first_step = (uint32_t)first_step;
    p.bank = s->ta_state;
    p.weights = s->clause_weights;
    p.literals = cfg->literals;
    p.n_types = g->number_of_node_types;
    p.C = d.C;
    p.LA = d.LA;
    p.B = d.B;
    p.K = d.K;
    p.T = cfg->threshold;
    p.negative = cfg->negative_clauses;
    p.boost = cfg->boost_true_positive_feedback;
    p.max_included = cfg->max_included_literals;
    p.filter = d.filter;
    p.thr16 = feedback_threshold(cfg->s[0]);
    p.k0 = key.k0;
    p.k1 = key.k1;
    p.q_thr = q_threshold(cfg->q, cfg->classes);
    p.class_sum = (unsigned long long *)w.class_sum;
    p.abort_flag = (uint32_t *)((unsigned long long *)w.class_sum + (size_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE);
    const WaitBound bound = wait_bound(dev);
    p.spin_limit = bound.spin_limit, p.wait_ticks = bound.wait_ticks, p.force_abort = bound.force_abort;
    // A run that gives up leaves the workgroups at different examples.  The bank and the weights
    // are kept as they were, so that a failed call leaves the model as it found it.
    const size_t bank_bytes = (size_t)d.C * d.LA * d.B * 4, weights_bytes = (size_t)d.K * d.C * 4;
    hipError_t e = hipMemcpyAsync(w.bank_backup, s->ta_state, bank_bytes, hipMemcpyDeviceToDevice, st);
    if (e == hipSuccess) e = hipMemcpyAsync(w.weights_backup, s->clause_weights, weights_bytes, hipMemcpyDeviceToDevice, st);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "keeping a copy of the model state: %s", hipGetErrorString(e));

    hipLaunchKernelGGL(k_fill_u64, dim3(blocks_for((int64_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE + 1, TPB)), dim3(TPB), 0, st,
                       (unsigned long long *)w.class_sum, (int64_t)0, 0ull, (int64_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE + 1);
    if (int rc = check_launch("fill")) return rc;
    void *args[] = {&p};
    profile_start("k_fit_persistent", st);
    e = hipLaunchCooperativeKernel(kernel, dim3(groups), dim3(FITP_BLOCK), args, (unsigned)lds, st);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "cooperative launch of the training kernel: %s", hipGetErrorString(e));
    profile_stop(st);
    uint32_t flag = 0;
    e = hipMemcpyAsync(&flag, p.abort_flag, 4, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "training kernel: %s", hipGetErrorString(e));
    if (flag != 0) {
        e = hipMemcpyAsync(s->ta_state, w.bank_backup, bank_bytes, hipMemcpyDeviceToDevice, st);
        if (e == hipSuccess) e = hipMemcpyAsync(s->clause_weights, w.weights_backup, weights_bytes, hipMemcpyDeviceToDevice, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess)
            return fail(GTM_ERR_HIP, "training kernel gave up waiting at its device-wide barrier (%d workgroups) and "
                                     "the model state could not be restored: %s", groups, hipGetErrorString(e));
        // The model is as it was.  A wait that really ran out (a GPU shared with other work, a very
        // large graph) is no reason to fail the call: the caller goes on with the launches per example,
        // which wait for nobody.  Only the forced give-up of the tests is reported.
        if (!p.force_abort) return GTM_OK;  // *done stays false
        return fail(GTM_ERR_HIP, "training kernel gave up waiting at its device-wide barrier (%d workgroups); "
                                 "the model state is as it was before the call", groups);
    }
    *done = true;
    return GTM_OK;
}

// `_fit`'s inner loop of a model with message layers as one cooperative launch (fit_deep_persistent.h).
// Returns GTM_OK with *done = false when this device or shape cannot run it, so that the caller
// falls back to the launches per example.  GTM_NO_DEEP_PERSISTENT_FIT (tuning aid) turns it off.
// With several clauses per workgroup the run is cut into launches of a few hundred to a few thousand examples
// and the clauses are dealt out anew before each (k_fit_deep_deal); *examples_done says how far the run got
// when a launch gave up (the model is then as it was before that launch).
int fit_deep_persistent(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, const TileGeom &tg,
                        const FitWs &w, const int32_t *encoded_Y, int first_example, int n_examples, uint64_t first_step,
                        hipStream_t st, bool *done, int *examples_done) {
    *done = false;
    *examples_done = 0;
    if (tune(T_NO_DEEP_PERSISTENT_FIT) || tune(T_NO_PERSISTENT_FIT) || cfg->depth < 2 || d.K > FITD_BLOCK) return GTM_OK;
    if (d.M % 32 != 0 || d.NC > 64) return GTM_OK;  // whole words of message bits; one lane per word of a truth row
    int dev = 0, coop = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return GTM_OK;
    if (hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev) != hipSuccess || !coop) return GTM_OK;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return GTM_OK;
    if (g->total_edges > 0 && (!g->number_of_graph_node_edges || !g->edge || !g->edge_index))
        return fail(GTM_ERR_INVALID, "graphs with edges need number_of_graph_node_edges, edge and edge_index");

    const int layers = cfg->depth - 1, MW = d.M / 32;
    int per_group = (d.C + cus - 1) / cus;
    if (const char *e = tune(T_FIT_DEEP_CLAUSES_PER_GROUP)) per_group = std::max(per_group, atoi(e));  // tuning aid
    const int groups = (d.C + per_group - 1) / per_group;
    const int NW = d.NC;
    const int rows_words = (cfg->literals + g->number_of_node_types + 1) * NW;
    // the edges of the run's examples: most per graph, largest type, stored node after node?
    uint32_t limits[3] = {0u, 0u, 0u};
    if (g->total_edges > 0) {
        hipLaunchKernelGGL(k_fill_i32, dim3(1), dim3(TPB), 0, st, (int32_t *)w.coop_got, (int64_t)3, 0);
        if (int rc = check_launch("fill")) return rc;
        hipLaunchKernelGGL(k_edge_limits, dim3(n_examples), dim3(256), 0, st, g->number_of_graph_nodes, g->node_index,
                           g->number_of_graph_node_edges, g->edge_index, g->edge, first_example, w.coop_got);
        if (int rc = check_launch("k_edge_limits")) return rc;
        hipError_t e = hipMemcpyAsync(limits, w.coop_got, sizeof(limits), hipMemcpyDeviceToHost, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "reading the edge limits: %s", hipGetErrorString(e));
        if (limits[2] != 0u || limits[1] >= (uint32_t)FITD_MAX_EDGE_TYPES || limits[0] > (1u << 20)) return GTM_OK;
    }
    const int edge_cap = (int)limits[0], edge_types = (int)limits[1] + 1;
    // automata, layer-0 rows and all received rows in LDS where they fit; else automata in memory, rows in
    // place and as wide a window of received rows as fits
    const size_t lds_cap = 158 * 1024;  // of 160 KiB; the kernel has a few words of its own
    bool big = tune(T_FIT_DEEP_IN_MEMORY) != nullptr;  // tuning aid: take the second layout anyway
    int window_rows = d.M;
    size_t lds = fit_deep_lds_words(false, cfg->depth, cfg->literals, per_group, d.LA, d.MC, d.MB, d.B, d.K, NW, rows_words, d.M, cfg->max_nodes,
                                    edge_cap, edge_types) * 4;
    if (lds > lds_cap) big = true;
    if (big) {
        if (const char *e = tune(T_FIT_DEEP_WINDOW_ROWS)) window_rows = std::max(32, std::min(d.M, atoi(e) / 32 * 32));
        for (;; window_rows = (window_rows / 2 + 31) / 32 * 32) {
            lds = fit_deep_lds_words(true, cfg->depth, cfg->literals, per_group, d.LA, d.MC, d.MB, d.B, d.K, NW, 0, window_rows, cfg->max_nodes,
                                     edge_cap, edge_types) * 4;
            if (lds <= lds_cap || window_rows == 32) break;
        }
        if (lds > lds_cap) return GTM_OK;
    }
    const int variant = (d.B <= 8 ? 0 : d.B <= 16 ? 1 : 2) + (big ? 3 : 0);
    const void *kernels[6] = {(const void *)k_fit_deep_persistent<8, false>,  (const void *)k_fit_deep_persistent<16, false>,
                              (const void *)k_fit_deep_persistent<32, false>, (const void *)k_fit_deep_persistent<8, true>,
                              (const void *)k_fit_deep_persistent<16, true>,  (const void *)k_fit_deep_persistent<32, true>};
    const void *kernel = kernels[variant];
    static thread_local size_t lds_set_of[6] = {48 * 1024, 48 * 1024, 48 * 1024, 48 * 1024, 48 * 1024, 48 * 1024};
    if (lds > lds_set_of[variant]) {
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            return GTM_OK;
        }
        lds_set_of[variant] = lds;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, FITD_BLOCK, lds) != hipSuccess || per_cu < 1 ||
        groups > per_cu * cus) {
        (void)hipGetLastError();
        return GTM_OK;
    }

    Key key = key_of(cfg);
    FitDeepParams p{};
    p.tiles = g->tiles;
    p.X = g->X;
    p.node_index = g->node_index;
    p.n_nodes = g->number_of_graph_nodes;
    p.n_edges = g->number_of_graph_node_edges;
    p.edge_index = g->edge_index;
    p.edge = g->edge;
    p.encoded_Y = encoded_Y;
    p.tg = tg;
    p.first_example = first_example;
    p.n_examples = n_examples;
    p.first_step = (uint32_t)first_step;
    p.bank[0] = s->ta_state;
    p.thr16[0] = feedback_threshold(cfg->s[0]);
    for (int l = 1; l < cfg->depth; ++l) {
        p.bank[l] = s->message_ta_state[l - 1];
        p.thr16[l] = feedback_threshold(cfg->s[l]);
    }
    p.weights = s->clause_weights;
    p.hv = s->hypervectors;
    p.depth = cfg->depth;
    p.literals = cfg->literals;
    p.n_types = g->number_of_node_types;
    p.C = d.C;
    p.LA = d.LA;
    p.MC = d.MC;
    p.MW = MW;
    p.M = d.M;
    p.MB = d.MB;
    p.B = d.B;
    p.K = d.K;
    p.T = cfg->threshold;
    p.negative = cfg->negative_clauses;
    p.boost = cfg->boost_true_positive_feedback;
    p.max_included = cfg->max_included_literals;
    p.has_edges = g->total_edges > 0;
    p.filter = d.filter;
    p.k0 = key.k0;
    p.k1 = key.k1;
    p.q_thr = q_threshold(cfg->q, cfg->classes);
    p.got = w.coop_got;
    p.vec = w.coop_vec;
    p.arrived = w.coop_arrived;
    p.class_sum = (unsigned long long *)w.class_sum;
    p.abort_flag = (uint32_t *)((unsigned long long *)w.class_sum + (size_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE);
    const WaitBound bound = wait_bound(dev);
    p.spin_limit = bound.spin_limit, p.wait_ticks = bound.wait_ticks, p.force_abort = bound.force_abort;
    p.clauses_per_group = per_group;
    p.NW = NW;
    p.rows_words = big ? 0 : rows_words;
    p.window_rows = window_rows;
    p.by_masks = (size_t)window_rows * NW >= (size_t)(1 + edge_types) * cfg->max_nodes && !tune(T_FIT_DEEP_NO_MASKS);
    p.order = g->tiles + tiles_words(tg) + (size_t)tg.rows * 2;
    p.max_nodes = cfg->max_nodes;
    p.edge_cap = edge_cap;
    p.edge_types = edge_types;

    // Several clauses per workgroup: the run in launches of 256, 512, ... 2,048 examples (early in training the
    // clauses change fastest), the clauses dealt out by their cost before each.  GTM_FIT_DEEP_CHUNK = n (tests):
    // launches of n examples; GTM_FIT_DEEP_NO_DEAL: one launch, clauses in order.
    const bool deal = per_group >= 2 && d.C <= FITD_DEAL_MAX && w.coop_perm && w.coop_cost &&
                      (size_t)groups * per_group <= (size_t)d.C + 2048 && !tune(T_FIT_DEEP_NO_DEAL);
    int chunk = deal ? 256 : n_examples;
    if (const char *e = tune(T_FIT_DEEP_CHUNK)) chunk = deal ? std::max(1, atoi(e)) : n_examples;
    const bool chunk_grows = deal && !tune(T_FIT_DEEP_CHUNK);
    static thread_local bool deal_lds_raised = false;
    if (deal && !deal_lds_raised) {
        if (hipFuncSetAttribute((const void *)k_fit_deep_deal, hipFuncAttributeMaxDynamicSharedMemorySize, FITD_DEAL_MAX * 8) !=
            hipSuccess)
            return fail(GTM_ERR_HIP, "raising the LDS limit of the dealing kernel");
        deal_lds_raised = true;
    }
    for (int at = 0; at < n_examples;) {
        const int n_now = std::min(chunk, n_examples - at);
        p.first_example = first_example + at;
        p.n_examples = n_now;
        p.first_step = (uint32_t)(first_step + (uint64_t)at);
        p.perm = nullptr;
        if (deal) {
            FitDeepBanks banks{};
            for (int l = 0; l < cfg->depth; ++l) banks.bank[l] = p.bank[l];
            hipLaunchKernelGGL(k_fit_deep_cost, dim3(blocks_for(d.C, TPB / 64)), dim3(TPB), 0, st, banks, cfg->depth, d.C, d.LA, d.MC,
                               d.B, w.coop_cost);
            if (int rc = check_launch("fit_deep_cost")) return rc;
            int pow2 = 1;
            while (pow2 < d.C) pow2 <<= 1;
            hipLaunchKernelGGL(k_fit_deep_deal, dim3(1), dim3(1024), (size_t)pow2 * 8, st, w.coop_cost, d.C, groups, per_group,
                               w.coop_perm);
            if (int rc = check_launch("fit_deep_deal")) return rc;
            p.perm = w.coop_perm;
        }
        // the exchange buffers start at zero; the model is kept as it was in case the run gives up
        hipLaunchKernelGGL(k_fill_u64, dim3(blocks_for((int64_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE + 1, TPB)), dim3(TPB), 0, st,
                           (unsigned long long *)w.class_sum, (int64_t)0, 0ull, (int64_t)d.K * 3 * FITP_SUM_PARTS * FITP_SUM_STRIDE + 1);
        if (int rc = check_launch("fill")) return rc;
        hipLaunchKernelGGL(k_fill_u64, dim3(blocks_for((int64_t)layers * FITD_PARTS * FITD_STRIDE, TPB)), dim3(TPB), 0, st,
                           w.coop_arrived, (int64_t)0, 0ull, (int64_t)layers * FITD_PARTS * FITD_STRIDE);
        if (int rc = check_launch("fill")) return rc;
        hipLaunchKernelGGL(k_fill_i32, dim3(blocks_for((int64_t)w.coop_words, TPB)), dim3(TPB), 0, st, (int32_t *)w.coop_got,
                           (int64_t)w.coop_words, 0);
        if (int rc = check_launch("fill")) return rc;
        const size_t bank0_bytes = (size_t)d.C * d.LA * d.B * 4, bankm_bytes = (size_t)d.C * d.MC * d.B * 4;
        const size_t weights_bytes = (size_t)d.K * d.C * 4;
        hipError_t e = hipMemcpyAsync(w.bank_backup, s->ta_state, bank0_bytes, hipMemcpyDeviceToDevice, st);
        for (int l = 0; l < layers && e == hipSuccess; ++l)
            e = hipMemcpyAsync((char *)w.bank_backup + bank0_bytes + (size_t)l * bankm_bytes, s->message_ta_state[l], bankm_bytes,
                               hipMemcpyDeviceToDevice, st);
        if (e == hipSuccess) e = hipMemcpyAsync(w.weights_backup, s->clause_weights, weights_bytes, hipMemcpyDeviceToDevice, st);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "keeping a copy of the model state: %s", hipGetErrorString(e));

#ifdef FITD_CLOCKS
        p.clocks = (unsigned long long *)w.bank_backup;  // (development builds only: an aborted run is not restored correctly)
#endif
        void *args[] = {&p};
        profile_start(big ? "k_fit_deep_persistent<in memory>" : "k_fit_deep_persistent", st);
        e = hipLaunchCooperativeKernel(kernel, dim3(groups), dim3(FITD_BLOCK), args, (unsigned)lds, st);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "cooperative launch of the training kernel: %s", hipGetErrorString(e));
        profile_stop(st);
        uint32_t flag = 0;
        e = hipMemcpyAsync(&flag, p.abort_flag, 4, hipMemcpyDeviceToHost, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return fail(GTM_ERR_HIP, "training kernel: %s", hipGetErrorString(e));
#ifdef FITD_CLOCKS
        {
            unsigned long long clk[16];
            (void)hipMemcpy(clk, w.bank_backup, sizeof(clk), hipMemcpyDeviceToHost);
            fprintf(stderr, "fitd clocks (us per example, %d groups):", groups);
            for (int k = 0; k < 13; ++k) fprintf(stderr, " %d:%.2f", k, clk[k] * 0.01 / n_examples);
            fprintf(stderr, "\n");
        }
#endif
        if (flag != 0) {
            e = hipMemcpyAsync(s->ta_state, w.bank_backup, bank0_bytes, hipMemcpyDeviceToDevice, st);
            for (int l = 0; l < layers && e == hipSuccess; ++l)
                e = hipMemcpyAsync(s->message_ta_state[l], (char *)w.bank_backup + bank0_bytes + (size_t)l * bankm_bytes, bankm_bytes,
                                   hipMemcpyDeviceToDevice, st);
            if (e == hipSuccess) e = hipMemcpyAsync(s->clause_weights, w.weights_backup, weights_bytes, hipMemcpyDeviceToDevice, st);
            if (e == hipSuccess) e = hipStreamSynchronize(st);
            if (e != hipSuccess)
                return fail(GTM_ERR_HIP, "training kernel gave up waiting at a device-wide barrier (%d workgroups) and the "
                                         "model state could not be restored: %s", groups, hipGetErrorString(e));
            if (!p.force_abort) return GTM_OK;  // as in fit_persistent: the launches per example take over
            return fail(GTM_ERR_HIP, "training kernel gave up waiting at a device-wide barrier (%d workgroups); "
                                     "the model state is as it was before the call", groups);
        }
        at += n_now;
        *examples_done = at;
        if (chunk_grows && chunk < 2048) chunk *= 2;
    }
    *done = true;
    return GTM_OK;
}

// `_fit`'s inner loop for a depth-1 model on a data set that has tiles: two
// launches per example (fit_fused.h).
int fit_on_tiles(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, const TileGeom &tg,
                 const FitWs &w, const int32_t *encoded_Y, int first_example, int n_examples, uint64_t first_step,
                 const uint32_t *h_n, const uint32_t *h_base, hipStream_t st) {
    hipLaunchKernelGGL(k_fill_i32, dim3(1), dim3(TPB), 0, st, w.class_sum, (int64_t)d.K * 2, 0);
    if (int rc = check_launch("fill")) return rc;
    const uint32_t *order = g->tiles + tiles_words(tg) + (size_t)tg.rows * 2;  // literals, rarest first
    Key key = key_of(cfg);
    const int n_types = g->number_of_node_types;
    const int cpb = d.LA >= TPB ? 1 : TPB / d.LA;
    const uint64_t q_thr = q_threshold(cfg->q, cfg->classes);
    const uint32_t thr16 = feedback_threshold(cfg->s[0]);
    // enough waves to spread the clauses over the chip, at least ~2 clauses per wave
    const int waves_per_block = FIT_EVAL_BLOCK / 64;
    int eval_blocks = (d.C + 2 * waves_per_block - 1) / (2 * waves_per_block);
    if (eval_blocks > 512) eval_blocks = 512;
    static thread_local size_t lds_set = 0;
    for (int i = 0; i < n_examples; ++i) {
        const int ex = first_example + i;
        const uint32_t step = (uint32_t)(first_step + (uint64_t)i);
        FitGraph fg = fit_graph_slot(tg, ex, (int)h_n[i]);
        int32_t *sum_now = w.class_sum + (size_t)(i & 1) * d.K, *sum_next = w.class_sum + (size_t)((i + 1) & 1) * d.K;
        size_t lds = (size_t)(cfg->literals + n_types + 1) * fg.words * 4;
        const bool stage = lds <= 96 * 1024;
        if (stage && lds > lds_set) {
            hipError_t e = hipFuncSetAttribute((const void *)k_fit_eval<true>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
            lds_set = lds;
        }
        if (i < Profile::MAX) profile_start(stage ? "k_fit_eval<true>" : "k_fit_eval<false>", st);
        if (stage)
            hipLaunchKernelGGL(k_fit_eval<true>, dim3(eval_blocks), dim3(FIT_EVAL_BLOCK), lds, st, g->tiles, tg, fg,
                               (int)h_n[i], cfg->literals, n_types, d.C, d.LA, d.B, d.K, d.NC, d.filter, s->ta_state,
                               s->clause_weights, key.k0, key.k1, step, 1, g->X + (int64_t)h_base[i] * d.LA, order, w.bitmap_a,
                               w.n_incl, w.clause_node, sum_now);
        else
            hipLaunchKernelGGL(k_fit_eval<false>, dim3(eval_blocks), dim3(FIT_EVAL_BLOCK), 0, st, g->tiles, tg, fg,
                               (int)h_n[i], cfg->literals, n_types, d.C, d.LA, d.B, d.K, d.NC, d.filter, s->ta_state,
                               s->clause_weights, key.k0, key.k1, step, 1, g->X + (int64_t)h_base[i] * d.LA, order, w.bitmap_a,
                               w.n_incl, w.clause_node, sum_now);
        if (int rc = check_launch("fit_eval")) return rc;
        if (i < Profile::MAX) profile_stop(st);
        FitBanks banks{};
        banks.n = 1;
        banks.total_chunks = d.LA;
        banks.bank[0] = s->ta_state;
        banks.rows[0] = g->X + (int64_t)h_base[i] * d.LA;
        banks.chunks[0] = d.LA;
        banks.thr16[0] = thr16;
        hipLaunchKernelGGL(k_fit_feedback, dim3(blocks_for(d.C, cpb)), dim3(TPB), (size_t)cpb * d.K * 4, st, banks,
                           s->clause_weights, sum_now, sum_next, encoded_Y + (int64_t)ex * d.K, d.C, d.B, d.K,
                           cfg->threshold, cfg->negative_clauses, cfg->boost_true_positive_feedback,
                           cfg->max_included_literals, q_thr, key.k0, key.k1, step, w.clause_node, w.n_incl, cpb);
        if (int rc = check_launch("fit_feedback")) return rc;
    }
    return GTM_OK;
}

// A small model with message layers on tiny graphs trains inside one workgroup (fit_small.h).
// Sets *done = false when the shape does not qualify.
int fit_small(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, const int32_t *encoded_Y,
              int first_example, int n_examples, uint64_t first_step, hipStream_t st, bool *done) {
    *done = false;
    if (tune(T_NO_SMALL_FIT)) return GTM_OK;
    if (cfg->depth < 2 || d.M % 32 != 0 || g->max_number_of_graph_nodes > FITS_MAX_NODES ||
        g->number_of_node_types < 1)
        return GTM_OK;
    const int MW = d.M / 32;
    const size_t lds = fit_small_lds_words(cfg->depth, d.C, d.LA, d.MC, MW, d.MB, d.B, d.K) * 4;
    if (lds > FITS_MAX_LDS_BYTES) return GTM_OK;
    if (g->total_edges > 0 && (!g->number_of_graph_node_edges || !g->edge || !g->edge_index))
        return fail(GTM_ERR_INVALID, "graphs with edges need number_of_graph_node_edges, edge and edge_index");
    Key key = key_of(cfg);
    FitSmallParams p{};
    p.X = g->X;
    p.node_type = g->node_type;
    p.node_index = g->node_index;
    p.n_nodes = g->number_of_graph_nodes;
    p.n_edges = g->number_of_graph_node_edges;
    p.edge_index = g->edge_index;
    p.edge = g->edge;
    p.encoded_Y = encoded_Y;
    p.first_example = first_example;
    p.n_examples = n_examples;
    p.first_step = (uint32_t)first_step;
    p.n_types = g->number_of_node_types;
    p.has_edges = g->total_edges > 0;
    p.bank[0] = s->ta_state;
    p.filter[0] = d.filter;
    p.thr16[0] = feedback_threshold(cfg->s[0]);
    for (int l = 1; l < cfg->depth; ++l) {
        p.bank[l] = s->message_ta_state[l - 1];
        p.filter[l] = d.mfilter;
        p.thr16[l] = feedback_threshold(cfg->s[l]);
    }
    p.weights = s->clause_weights;
    p.hv = s->hypervectors;
    p.depth = cfg->depth;
    p.C = d.C;
    p.LA = d.LA;
    p.MC = d.MC;
    p.MW = MW;
    p.MB = d.MB;
    p.B = d.B;
    p.K = d.K;
    p.T = cfg->threshold;
    p.negative = cfg->negative_clauses;
    p.boost = cfg->boost_true_positive_feedback;
    p.max_included = cfg->max_included_literals;
    p.k0 = key.k0;
    p.k1 = key.k1;
    p.q_thr = q_threshold(cfg->q, cfg->classes);
    static thread_local size_t lds_set = 48 * 1024;
    if (lds > lds_set) {
        if (hipFuncSetAttribute((const void *)k_fit_small, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
            hipSuccess) {
            (void)hipGetLastError();
            return GTM_OK;
        }
        lds_set = lds;
    }
    profile_start("k_fit_small", st);
    hipLaunchKernelGGL(k_fit_small, dim3(1), dim3(FITS_BLOCK), lds, st, p);
    profile_stop(st);
    if (int rc = check_launch("fit_small")) return rc;
    *done = true;
    return GTM_OK;
}

// One training step of a model with message layers (tm.py:669-747) in 2 + 4 launches per layer:
// layer 0 on the graph's tile rows, then per message layer the messages (blank, scatter,
// literal-major copy) and the conditional evaluation, then one feedback kernel over all banks.
int fit_deep_on_tiles(const Dims &d, const gtm_config *cfg, const gtm_graphs *g, const gtm_state *s, const TileGeom &tg,
                      const FitWs &w, const int32_t *encoded_Y, int first_example, int n_examples, uint64_t first_step,
                      const uint32_t *h_n, const uint32_t *h_base, hipStream_t st) {
    hipLaunchKernelGGL(k_fill_i32, dim3(1), dim3(TPB), 0, st, w.class_sum, (int64_t)d.K * 2, 0);
    if (int rc = check_launch("fill")) return rc;
    if (g->total_edges > 0 && (!g->number_of_graph_node_edges || !g->edge || !g->edge_index))
        return fail(GTM_ERR_INVALID, "graphs with edges need number_of_graph_node_edges, edge and edge_index");
    const uint32_t *order = g->tiles + tiles_words(tg) + (size_t)tg.rows * 2;  // literals, rarest first
    Key key = key_of(cfg);
    const int n_types = g->number_of_node_types;
    const int layers = cfg->depth - 1;
    const int per_clause = d.LA + layers * d.MC;
    const int cpb = per_clause >= TPB ? 1 : TPB / per_clause;
    const uint64_t q_thr = q_threshold(cfg->q, cfg->classes);
    const int waves_per_block = FIT_EVAL_BLOCK / 64;
    // one clause per wave while the chip has room (the evaluation is a chain of memory round trips)
    int eval_blocks = (d.C + waves_per_block - 1) / waves_per_block;
    if (eval_blocks > 2048) eval_blocks = 2048;
    static thread_local size_t lds_set = 0;
    // Messages by per-node bit vectors (fit_deep.h) when MESSAGE_SIZE is a multiple of 32 and the
    // graph is big enough for the saved atomics to pay for the extra pass.
    const int MW = (d.M + 31) / 32;
    const bool factored = d.M % 32 == 0 && (size_t)32 * MW * 4 <= 48 * 1024;
    const char *fm = tune(T_FIT_FACTOR_MIN);  // clauses x nodes from which that path is taken (tuning aid)
    const int64_t factor_min = fm ? atoll(fm) : 32768;
    if (factored) {
        const int64_t vector_words = (int64_t)cfg->max_nodes * MW;
        for (uint32_t *p : {w.sent, w.got}) {
            hipLaunchKernelGGL(k_fill_i32, dim3(blocks_for(vector_words, TPB)), dim3(TPB), 0, st, (int32_t *)p,
                               vector_words, 0);
            if (int rc = check_launch("fill")) return rc;
        }
    }
    for (int i = 0; i < n_examples; ++i) {
        const int ex = first_example + i;
        const int n_nodes = (int)h_n[i];
        const uint32_t step = (uint32_t)(first_step + (uint64_t)i);
        FitGraph fg = fit_graph_slot(tg, ex, n_nodes);
        int32_t *sum_now = w.class_sum + (size_t)(i & 1) * d.K, *sum_next = w.class_sum + (size_t)((i + 1) & 1) * d.K;
        size_t lds = (size_t)(cfg->literals + n_types + 1) * fg.words * 4;
        const bool stage = lds <= 96 * 1024;
        if (stage && lds > lds_set) {
            hipError_t e = hipFuncSetAttribute((const void *)k_fit_eval<true>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return fail(GTM_ERR_HIP, "raising the LDS limit to %zu: %s", lds, hipGetErrorString(e));
            lds_set = lds;
        }
        if (stage)
            hipLaunchKernelGGL(k_fit_eval<true>, dim3(eval_blocks), dim3(FIT_EVAL_BLOCK), lds, st, g->tiles, tg, fg,
                               n_nodes, cfg->literals, n_types, d.C, d.LA, d.B, d.K, d.NC, d.filter, s->ta_state,
                               s->clause_weights, key.k0, key.k1, step, 0, g->X + (int64_t)h_base[i] * d.LA, order, w.bitmap_a,
                               w.n_incl, w.clause_node, sum_now);
        else
            hipLaunchKernelGGL(k_fit_eval<false>, dim3(eval_blocks), dim3(FIT_EVAL_BLOCK), 0, st, g->tiles, tg, fg,
                               n_nodes, cfg->literals, n_types, d.C, d.LA, d.B, d.K, d.NC, d.filter, s->ta_state,
                               s->clause_weights, key.k0, key.k1, step, 0, g->X + (int64_t)h_base[i] * d.LA, order, w.bitmap_a,
                               w.n_incl, w.clause_node, sum_now);
        if (int rc = check_launch("fit_eval")) return rc;
        uint32_t *cur = w.bitmap_a, *nxt = w.bitmap_b;
        const int words = n_nodes == 0 ? 1 : (n_nodes - 1) / 32 + 1;
        for (int l = 0; l < layers; ++l) {
            uint32_t *cx = w.clause_X[l];
            if (factored && (int64_t)d.C * n_nodes >= factor_min) {
                if (n_nodes > 0 && g->total_edges > 0) {  // without edges nothing is received: the messages stay blank
                    // with every clause in one block, that block also sends its vectors along the edges
                    const int clause_blocks = (d.C + FIT_NODE_MESSAGES_CLAUSES - 1) / FIT_NODE_MESSAGES_CLAUSES;
                    const bool and_edges = clause_blocks == 1;
                    const uint32_t *no_edges = nullptr;
                    hipLaunchKernelGGL(k_fit_node_messages, dim3(words, clause_blocks), dim3(FIT_NODE_MESSAGES_BLOCK),
                                       (size_t)32 * (MW | 1) * 4, st, cur, d.C, d.NC, n_nodes, s->hypervectors, d.MB, MW,
                                       w.sent, and_edges ? g->number_of_graph_node_edges + h_base[i] : no_edges,
                                       and_edges ? g->edge_index + h_base[i] : no_edges, g->edge, w.got);
                    if (int rc = check_launch("fit_node_messages")) return rc;
                    if (!and_edges) {
                        hipLaunchKernelGGL(k_fit_edge_messages, dim3(blocks_for((int64_t)n_nodes * MW, TPB)), dim3(TPB), 0,
                                           st, w.sent, n_nodes, MW, g->number_of_graph_node_edges + h_base[i],
                                           g->edge_index + h_base[i], g->edge, w.got);
                        if (int rc = check_launch("fit_edge_messages")) return rc;
                    }
                }
                hipLaunchKernelGGL(k_fit_pack_messages, dim3(MW, w.message_row_words / 2), dim3(64), 0, st, w.sent, w.got,
                                   n_nodes, MW, w.message_row_words, cx, w.message_rows);
                if (int rc = check_launch("fit_pack_messages")) return rc;
            } else {
                if (n_nodes > 0) {
                    const int64_t message_words = (int64_t)n_nodes * d.MC;
                    hipLaunchKernelGGL(k_messages_blank, dim3(blocks_for(message_words, TPB)), dim3(TPB), 0, st, cx,
                                       message_words, d.MC, d.M);
                    if (int rc = check_launch("messages_blank")) return rc;
                    if (g->total_edges > 0) {
                        const int64_t pairs = (int64_t)d.C * n_nodes;
                        hipLaunchKernelGGL(k_fit_scatter_messages, dim3(blocks_for(pairs, FIT_SCATTER_BLOCK)),
                                           dim3(FIT_SCATTER_BLOCK), 0, st, cur, d.C, d.NC, n_nodes, s->hypervectors, d.MB,
                                           d.M, d.MC, g->number_of_graph_node_edges + h_base[i],
                                           g->edge_index + h_base[i], g->edge, cx);
                        if (int rc = check_launch("fit_scatter_messages")) return rc;
                    }
                }
                hipLaunchKernelGGL(k_fit_message_rows, dim3((d.M + 31) / 32, w.message_row_words / 2), dim3(64), 0, st,
                                   cx, n_nodes, d.M, d.MC, w.message_row_words, w.message_rows);
                if (int rc = check_launch("fit_message_rows")) return rc;
            }
            // waves per clause: one per block of 64 nodes while the chip has room for that many
            int eval_waves = (n_nodes + 63) / 64;
            eval_waves = eval_waves < 4 ? 4 : eval_waves > FIT_MESSAGE_EVAL_BLOCK / 64 ? FIT_MESSAGE_EVAL_BLOCK / 64 : eval_waves;
            if ((int64_t)d.C * eval_waves > 16384) eval_waves = 4;
            hipLaunchKernelGGL(k_fit_message_eval, dim3(d.C < 4096 ? d.C : 4096), dim3(eval_waves * 64), 0, st, w.message_rows,
                               w.message_row_words, cx, words, n_nodes, d.M, d.C, d.MC, d.B, d.K, d.NC, d.mfilter,
                               s->message_ta_state[l], s->clause_weights, key.k0, key.k1, step, l == layers - 1 ? 1 : 0,
                               cur, nxt, w.n_incl, w.clause_node, sum_now);
            if (int rc = check_launch("fit_message_eval")) return rc;
            uint32_t *t = cur;
            cur = nxt;
            nxt = t;
        }
        FitBanks banks{};
        banks.n = cfg->depth;
        banks.total_chunks = per_clause;
        banks.bank[0] = s->ta_state;
        banks.rows[0] = g->X + (int64_t)h_base[i] * d.LA;
        banks.chunks[0] = d.LA;
        banks.thr16[0] = feedback_threshold(cfg->s[0]);
        for (int l = 0; l < layers; ++l) {
            banks.bank[l + 1] = s->message_ta_state[l];
            banks.rows[l + 1] = w.clause_X[l];
            banks.chunks[l + 1] = d.MC;
            banks.thr16[l + 1] = feedback_threshold(cfg->s[l + 1]);
        }
        hipLaunchKernelGGL(k_fit_feedback, dim3(blocks_for(d.C, cpb)), dim3(TPB), (size_t)cpb * d.K * 4, st, banks,
                           s->clause_weights, sum_now, sum_next, encoded_Y + (int64_t)ex * d.K, d.C, d.B, d.K,
                           cfg->threshold, cfg->negative_clauses, cfg->boost_true_positive_feedback,
                           cfg->max_included_literals, q_thr, key.k0, key.k1, step, w.clause_node, w.n_incl, cpb);
        if (int rc = check_launch("fit_feedback")) return rc;
    }
    return GTM_OK;
}

}  // namespace

extern "C" {

size_t gtm_fit_workspace_bytes(const gtm_config *cfg, const gtm_graphs *graphs) {
    Dims d;
    if (validate(cfg, &d)) return 0;
    (void)graphs;
    return carve_fit(d, cfg, nullptr).bytes;
}

int gtm_fit(const gtm_config *cfg, const gtm_graphs *graphs, const gtm_state *state, const int32_t *encoded_Y,
            int32_t first_example, int32_t n_examples, uint64_t first_step, void *workspace,
            size_t workspace_bytes, void *stream) {
    Dims d;
    if (int rc = validate(cfg, &d)) return rc;
    if (int rc = validate_graphs(cfg, graphs, first_example, n_examples)) return rc;
    if (int rc = validate_state(cfg, state)) return rc;
    if (!encoded_Y) return fail(GTM_ERR_INVALID, "encoded_Y is NULL");
    FitWs w = carve_fit(d, cfg, (char *)workspace);
    if (!workspace || workspace_bytes < w.bytes)
        return fail(GTM_ERR_INVALID, "workspace of %zu bytes needed, %zu given", w.bytes, workspace_bytes);
    if (n_examples == 0) return GTM_OK;
    hipStream_t st = (hipStream_t)stream;
    // node counts and offsets of the examples, read once
    std::string host((size_t)n_examples * 8, '\0');
    uint32_t *h_n = (uint32_t *)host.data();
    uint32_t *h_base = h_n + n_examples;
    hipError_t e = hipMemcpyAsync(h_n, graphs->number_of_graph_nodes + first_example, (size_t)n_examples * 4,
                                  hipMemcpyDeviceToHost, st);
    if (e == hipSuccess)
        e = hipMemcpyAsync(h_base, graphs->node_index + first_example, (size_t)n_examples * 4, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(GTM_ERR_HIP, "reading graph sizes: %s", hipGetErrorString(e));

    if (graphs->tiles) {
        TileGeom tg = geometry_for(cfg, graphs, d.K);
        if (tg.ok)
            if (int rc = check_tiles(tg, cfg, graphs)) return rc;
    }
    if (cfg->depth == 1 && graphs->tiles) {
        TileGeom tg = geometry_for(cfg, graphs, d.K);
        if (tg.ok && tg.slot_words <= 64) {  // one lane per word of the graph's slot
            bool done = false;
            if (int rc = fit_persistent(d, cfg, graphs, state, tg, w, encoded_Y, first_example, n_examples, first_step,
                                        st, &done))
                return rc;
            if (done) return GTM_OK;
            return fit_on_tiles(d, cfg, graphs, state, tg, w, encoded_Y, first_example, n_examples, first_step, h_n,
                                h_base, st);
        }
    }
    if (cfg->depth > 1) {
        bool done = false;
        if (int rc = fit_small(d, cfg, graphs, state, encoded_Y, first_example, n_examples, first_step, st, &done)) return rc;
        if (done) return GTM_OK;
    }
    if (cfg->depth > 1 && graphs->tiles && graphs->number_of_node_types >= 1 && !tune(T_NO_DEEP_FIT)) {
        TileGeom tg = geometry_for(cfg, graphs, d.K);
        if (tg.ok && tg.slot_words <= 64 && cfg->max_nodes <= 2048) {  // one lane per word of the graph's nodes
            bool done = false;
            int so_far = 0;  // examples that launches which did not give up have trained on
            if (int rc = fit_deep_persistent(d, cfg, graphs, state, tg, w, encoded_Y, first_example, n_examples, first_step, st,
                                             &done, &so_far))
                return rc;
            if (done) return GTM_OK;
            first_example += so_far, n_examples -= so_far, first_step += (uint64_t)so_far, h_n += so_far, h_base += so_far;
        }
        if (tg.ok && tg.slot_words <= 64 && cfg->max_nodes <= 2048)
            return fit_deep_on_tiles(d, cfg, graphs, state, tg, w, encoded_Y, first_example, n_examples, first_step, h_n,
                                     h_base, st);
    }
    for (int i = 0; i < n_examples; ++i) {
        int ex = first_example + i;
        uint64_t step = first_step + (uint64_t)i;
        uint32_t *final_bitmap = nullptr;
        if (int rc = run_evaluate(d, cfg, graphs, state, ex, 1, w.inc_t, w.bitmap_a, w.bitmap_b, w.clause_X, true,
                                  w.n_incl, w.class_sum, &final_bitmap, st))
            return rc;
        if (int rc = op_select_clause_node(d, cfg, (int)h_n[i], step, final_bitmap, w.clause_node, st)) return rc;
        if (int rc = op_select_clause_updates(d, cfg, step, state->clause_weights, w.class_sum,
                                              encoded_Y + (int64_t)ex * d.K, w.clause_node, w.update, st))
            return rc;
        if (int rc = op_update(d, cfg, step, 0, state->ta_state, d.LA, w.clause_node, w.n_incl,
                               graphs->X + (int64_t)h_base[i] * d.LA, w.update, st))
            return rc;
        for (int layer = 0; layer < cfg->depth - 1; ++layer)
            if (int rc = op_update(d, cfg, step, layer + 1, state->message_ta_state[layer], d.MC, w.clause_node,
                                   w.n_incl, w.clause_X[layer], w.update, st))
                return rc;
    }
    return GTM_OK;
}

}  // extern "C"
