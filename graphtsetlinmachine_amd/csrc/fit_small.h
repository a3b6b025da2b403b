// A run of training examples (the loop at tm.py:669-747) of a SMALL model with
// message layers on TINY graphs (at most 64 nodes, MESSAGE_SIZE a multiple of
// 32) as one launch of one workgroup: the automata of every bank, the weights
// and everything a step produces live in LDS, and the phases of a step are
// separated by workgroup barriers only.  At this size a step is a chain of
// dependent latencies, not work: a dozen barriers instead of six kernel
// launches per example.
//
// Per example:
//   load     the graph's literal words and node types                  -> LDS
//   layer 0  K1: wave per clause, lane = node: (include & ~X[node]) == 0 and the
//            node-type gate (kernels.py:443-466)
//   per message layer
//            K3-K5: per-node bit vectors of what the true clauses send
//            (kernels.py:565-588), rotated along the edges, packed with their
//            negations; K2: wave per clause, lane = node, against the message
//            bank's include words (kernels.py:505-527)
//   K7, K6   node pick and class sums (kernels.py:319-354, :279-317)
//   K8       feedback decision, weight update (kernels.py:356-405)
//   K9, K10  Type I / II on every bank (kernels.py:98-242)
// The random numbers are the same counter-based ones as everywhere else, so the
// result equals the other training paths bit for bit.
#pragma once

constexpr int FITS_BLOCK = 256;
constexpr int FITS_MAX_NODES = 64;
constexpr size_t FITS_MAX_LDS_BYTES = 128 * 1024;  // of the 160 KB a workgroup can have

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
inline size_t fit_small_lds_words(int depth, int C, int LA, int MC, int MW, int B, int K) {
    const size_t banks = (size_t)C * (LA + (size_t)(depth - 1) * MC) * B;
    return banks + (size_t)K * C                              // weights
           + (size_t)FITS_MAX_NODES * LA + FITS_MAX_NODES     // X rows, node types
           + 2 * (size_t)C * 2                                // truth of two layers, 2 words per clause
           + 2 * (size_t)FITS_MAX_NODES * MW                  // sent, got
           + (size_t)(depth - 1) * FITS_MAX_NODES * MC        // packed messages per layer
           + (size_t)K + 2 * (size_t)C + (size_t)C * K;       // class sums, picked node, include count, updates
}

__global__ __launch_bounds__(FITS_BLOCK) void k_fit_small(FitSmallParams p) {
    extern __shared__ __align__(16) uint32_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int WAVES = FITS_BLOCK / 64;
    const int C = p.C, LA = p.LA, MC = p.MC, MW = p.MW, B = p.B, K = p.K, layers = p.depth - 1;

    // LDS carve-up: bank 0, then the message banks (all of one size), then the rest
    const size_t bank0_words = (size_t)C * LA * B, message_bank_words = (size_t)C * MC * B;
    auto bank_of = [&](int l) { return l == 0 ? lds : lds + bank0_words + (size_t)(l - 1) * message_bank_words; };
    int32_t *wts = (int32_t *)(lds + bank0_words + (size_t)layers * message_bank_words);  // [K][C]
    uint32_t *x_rows = (uint32_t *)(wts + K * C);  // [nodes][LA]
    uint32_t *types = x_rows + FITS_MAX_NODES * LA;
    uint32_t *truth[2] = {types + FITS_MAX_NODES, types + FITS_MAX_NODES + 2 * C};  // [C][2]
    uint32_t *sent = truth[1] + 2 * C;             // [nodes][MW]
    uint32_t *got = sent + FITS_MAX_NODES * MW;    // [nodes][MW]
    uint32_t *packed = got + FITS_MAX_NODES * MW;  // [layers][nodes][MC]
    int32_t *sums = (int32_t *)(packed + (size_t)layers * FITS_MAX_NODES * MC);  // [K]
    int32_t *node_of = sums + K;                   // [C]
    int32_t *incl_of = node_of + C;                // [C]
    int32_t *upd = incl_of + C;                    // [C][K]

    // state -> LDS
    for (int l = 0; l < p.depth; ++l) {
        uint32_t *dst = bank_of(l);
        const uint32_t *src = p.bank[l];
        for (int i = tid; i < C * (l == 0 ? LA : MC) * B; i += FITS_BLOCK) dst[i] = src[i];
    }
    for (int i = tid; i < K * C; i += FITS_BLOCK) wts[i] = p.weights[i];
    __syncthreads();

    for (int i = 0; i < p.n_examples; ++i) {
        const int ex = p.first_example + i;
        const uint32_t step = p.first_step + (uint32_t)i;
        const int n_nodes = (int)p.n_nodes[ex];
        const int64_t base = p.node_index[ex];
        const int words = n_nodes == 0 ? 1 : (n_nodes - 1) / 32 + 1;  // truth words in use (1 or 2)

        // ---- the graph -> LDS
        for (int j = tid; j < n_nodes * LA; j += FITS_BLOCK) x_rows[j] = p.X[base * LA + j];
        for (int j = tid; j < n_nodes; j += FITS_BLOCK) types[j] = p.node_type[base + j];
        for (int k = tid; k < K; k += FITS_BLOCK) sums[k] = 0;
        __syncthreads();

        // ---- layer 0 (K1): lane = node
        uint32_t *cur = truth[0], *nxt = truth[1];
        for (int c = wave; c < C; c += WAVES) {
            const uint32_t *inc = lds + (size_t)c * LA * B + (B - 1);
            bool ok = lane < n_nodes && (int)types[lane < n_nodes ? lane : 0] == c % p.n_types;
            int included = 0;
            for (int w = 0; w < LA; ++w) {
                uint32_t word = inc[w * B];
                if (w == LA - 1) word &= p.filter[0];
                included += __popc(word);
                ok = ok && (word & ~x_rows[(lane < n_nodes ? lane : 0) * LA + w]) == 0;
            }
            const unsigned long long t = __ballot(ok);
            if (lane == 0) {
                // a graph without nodes: the reference's arithmetic leaves every clause true (kernels.py:289-295)
                cur[2 * c] = n_nodes == 0 ? 0xFFFFFFFFu : (uint32_t)t;
                cur[2 * c + 1] = (uint32_t)(t >> 32);
                incl_of[c] = included;
            }
        }
        __syncthreads();

        // ---- message layers
        for (int l = 0; l < layers; ++l) {
            uint32_t *cx = packed + (size_t)l * FITS_MAX_NODES * MC;
            for (int j = tid; j < 2 * FITS_MAX_NODES * MW; j += FITS_BLOCK) sent[j] = 0u;  // sent and got are adjacent
            __syncthreads();
            // what each node sends: the hypervector bits of the clauses true at it
            for (int j = tid; j < C * n_nodes; j += FITS_BLOCK) {
                const int c = j / n_nodes, n = j - c * n_nodes;
                if ((cur[2 * c + (n >> 5)] >> (n & 31)) & 1u)
                    for (int b = 0; b < p.MB; ++b) {
                        const uint32_t h = p.hv[c * p.MB + b];
                        atomicOr(&sent[n * MW + (h >> 5)], 1u << (h & 31));
                    }
            }
            __syncthreads();
            // along every edge: the vector rotated by the edge type (bit p of the result is bit (p - type) mod M)
            if (p.has_edges)
                for (int j = tid; j < n_nodes * MW; j += FITS_BLOCK) {
                    const int n = j / MW, jw = j - n * MW;
                    const uint32_t ne = p.n_edges[base + n];
                    const int64_t e0 = p.edge_index[base + n];
                    const uint32_t *v = sent + n * MW;
                    for (uint32_t e = 0; e < ne; ++e) {
                        const uint32_t dst = p.edge[(e0 + e) * 2], shift = p.edge[(e0 + e) * 2 + 1] % (uint32_t)(MW * 32);
                        const int q = (int)(shift >> 5), r = (int)(shift & 31u);
                        const int a = (jw - q + MW) % MW, below = (a - 1 + MW) % MW;
                        const uint32_t word = r ? (v[a] << r) | (v[below] >> (32 - r)) : v[a];
                        if (word) atomicOr(&got[dst * MW + jw], word);
                    }
                }
            __syncthreads();
            // packed literals: the messages, then their negations
            for (int j = tid; j < n_nodes * MW; j += FITS_BLOCK) {
                const int n = j / MW, jw = j - n * MW;
                const uint32_t word = got[j];
                cx[n * MC + jw] = word;
                cx[n * MC + MW + jw] = ~word;
            }
            __syncthreads();
            // K2: lane = node
            for (int c = wave; c < C; c += WAVES) {
                const uint32_t *inc = bank_of(l + 1) + (size_t)c * MC * B + (B - 1);
                const int n = lane < n_nodes ? lane : 0;
                bool ok = lane < n_nodes && ((cur[2 * c + (n >> 5)] >> (n & 31)) & 1u);
                int included = 0;
                for (int w = 0; w < MC; ++w) {
                    uint32_t word = inc[w * B];
                    if (w == MC - 1) word &= p.filter[l + 1];
                    included += __popc(word);
                    ok = ok && (word & ~cx[n * MC + w]) == 0;
                }
                const unsigned long long t = __ballot(ok);
                if (lane == 0) {
                    nxt[2 * c] = n_nodes == 0 ? 0xFFFFFFFFu : (uint32_t)t;
                    nxt[2 * c + 1] = (uint32_t)(t >> 32);
                    incl_of[c] += included;
                }
            }
            __syncthreads();
            uint32_t *swap = cur;
            cur = nxt;
            nxt = swap;
        }

        // ---- K7 + K6: node pick and class sums, one thread per clause
        for (int c = tid; c < C; c += FITS_BLOCK) {
            const uint32_t lo = cur[2 * c], hi = words > 1 ? cur[2 * c + 1] : 0u;
            int node = -1;
            bool fired;
            if (n_nodes == 0) {
                fired = true;
            } else {
                const int count = __popc(lo) + __popc(hi);
                fired = count > 0;
                if (fired) {
                    philox_out r = philox4x32_10((uint32_t)c, 0u, step, GTM_TAG_CLAUSE_NODE, p.k0, p.k1);
                    int pick = (int)(((uint64_t)r.v[0] * (uint64_t)count) >> 32);
                    unsigned long long bits = ((unsigned long long)hi << 32) | lo;
                    for (int j = 0; j < pick; ++j) bits &= bits - 1;
                    node = __ffsll((long long)bits) - 1;
                }
            }
            node_of[c] = node;
            if (fired)
                for (int k = 0; k < K; ++k) atomicAdd(&sums[k], wts[k * C + c]);
        }
        __syncthreads();

        // ---- K8: feedback decision and weight update, one thread per (clause, class)
        const int32_t *y = p.encoded_Y + (int64_t)ex * K;
        for (int j = tid; j < C * K; j += FITS_BLOCK) {
            const int c = j / K, k = j - c * K;
            int cs = sums[k];
            cs = cs > p.T ? p.T : (cs < -p.T ? -p.T : cs);
            const int yk = y[k];
            const int target = 1 - 2 * (cs > yk);
            int w = wts[k * C + c];
            const int sign = (w >= 0) - (w < 0);
            int err = yk - cs;
            err = err < 0 ? -err : err;
            philox_out r = philox4x32_10((uint32_t)c, (uint32_t)k, step, GTM_TAG_CLAUSE_UPDATES, p.k0, p.k1);
            const bool skip = (target == -1 && (uint64_t)r.v[0] >= p.q_thr) ||
                              ((uint64_t)r.v[1] * (uint64_t)(2 * (int64_t)p.T) >= ((uint64_t)err << 32));
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
        __syncthreads();

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
            const uint32_t *rows = l == 0 ? x_rows : packed + (size_t)(l - 1) * FITS_MAX_NODES * MC;
            const uint32_t x = fired ? rows[node * chunks + w] : 0u;
            uint32_t thr16 = p.thr16[0];
#pragma unroll
            for (int t = 1; t < GTM_MAX_DEPTH; ++t)
                if (t == l) thr16 = p.thr16[t];
            feedback_word_any(bank_of(l) + ((size_t)c * chunks + w) * B, B, K, u_of, 1, fired, within, p.boost, x, p.k0, p.k1,
                              (uint32_t)c, (uint32_t)w, step, (uint32_t)l, thr16);
        }
        __syncthreads();
    }

    // state -> global memory
    for (int l = 0; l < p.depth; ++l) {
        const uint32_t *src = bank_of(l);
        uint32_t *dst = p.bank[l];
        for (int i = tid; i < C * (l == 0 ? LA : MC) * B; i += FITS_BLOCK) dst[i] = src[i];
    }
    for (int i = tid; i < K * C; i += FITS_BLOCK) p.weights[i] = wts[i];
}
