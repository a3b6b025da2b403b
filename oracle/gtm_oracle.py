"""CPU NumPy oracle for the Graph Tsetlin Machine hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
module; it is the checker that the HIP path is compared against (tests, the
smoke check and the benchmark's CPU-baseline leg).  It restates, function by
function, what the reference's CUDA kernels compute
(GraphTsetlinMachine/kernels.py) and how the reference's driver sequences
them (GraphTsetlinMachine/tm.py:563-812), on the reference's own memory
layouts:

* ``ta_state``  uint32 ``[CLAUSES][chunks][STATE_BITS]``, bit-sliced: bit ``b``
  of the automaton of literal ``k`` is bit ``k % 32`` of word
  ``[clause][k // 32][b]``; plane ``STATE_BITS-1`` is the include mask.
* ``clause_weights`` int32 ``[CLASSES][CLAUSES]``.
* clause/node truth bitmap uint32 ``[CLAUSES][NODE_CHUNKS]``, node ``n`` at bit
  ``n % 32`` of word ``n // 32``.
* packed message literals uint32 ``[nodes][MESSAGE_CHUNKS]``.

Random numbers.  The reference draws from cuRAND XORWOW states indexed by the
physical thread id, so its stream depends on the launch shape and cannot be
restated (parity unpinned for the stream itself; only the distributions are
contractual).  This oracle and the HIP kernels instead share a counter-based
generator, Philox4x32-10 (Salmon et al., SC'11), keyed by the model seed and
addressed by the logical site ``(clause, class/word, training step, purpose)``,
so both produce the same decisions whatever the launch shape.  ``philox4x32``
is pinned by the published Random123 known-answer vectors.

Pinned by tests/test_oracle_*.py: brute-force literal-level evaluation,
set-semantics messages, closed-form saturating counters, exhaustive feedback
cases, Philox known answers.  Parity unpinned: none of the deterministic
functions; the random stream as explained above.
"""

from dataclasses import dataclass, field

import numpy as np

U32 = np.uint32
U64 = np.uint64
MASK32 = 0xFFFFFFFF

# purposes of a random draw (low byte of counter word 3)
TAG_PREPARE = 1
TAG_CLAUSE_NODE = 2
TAG_CLAUSE_UPDATES = 3
TAG_FEEDBACK = 4

INT_MAX = 2147483647


# --------------------------------------------------------------------------
# configuration: the compile-time macros of the reference
# (tm.py:438-464, kernels.py:24-48)
# --------------------------------------------------------------------------


@dataclass
class Config:
    classes: int
    clauses: int
    literals: int
    state_bits: int = 8
    boost_true_positive_feedback: int = 1
    threshold: int = 100
    q: float = 1.0
    max_included_literals: int = None
    negative_clauses: int = 1
    max_nodes: int = 1
    message_size: int = 256
    message_bits: int = 2
    la_chunks: int = field(init=False)
    message_literals: int = field(init=False)
    message_chunks: int = field(init=False)
    node_chunks: int = field(init=False)
    filter: int = field(init=False)
    message_filter: int = field(init=False)

    def __post_init__(self):
        if self.max_included_literals is None:
            self.max_included_literals = self.literals
        self.la_chunks = (self.literals - 1) // 32 + 1
        self.message_literals = self.message_size * 2
        self.message_chunks = (self.message_literals - 1) // 32 + 1
        self.node_chunks = (self.max_nodes - 1) // 32 + 1
        self.filter = _tail_filter(self.literals)
        self.message_filter = _tail_filter(self.message_literals)


def _tail_filter(n_bits):
    """kernels.py:37-47: mask of the valid bits of the last word."""
    r = n_bits % 32
    return MASK32 if r == 0 else (~(MASK32 << r)) & MASK32


def feedback_threshold(s):
    """A Type I feedback bit is set when a 16-bit uniform is below this.

    Stands for ``curand_uniform <= 1.0/s`` (kernels.py:115,159): probability
    1/s, and exactly 1 for s = 1."""
    return min(65536, int(65536.0 / float(s)))


def q_threshold(q, classes):
    """``uniform <= q / max(1, CLASSES-1)`` (kernels.py:384) as a 32-bit
    integer comparison ``r < threshold`` with threshold in [0, 2**32]."""
    p = float(q) / max(1, classes - 1)
    p = min(1.0, max(0.0, p))
    return int(p * 4294967296.0)


# --------------------------------------------------------------------------
# Philox4x32-10
# --------------------------------------------------------------------------

_PHILOX_M0 = U64(0xD2511F53)
_PHILOX_M1 = U64(0xCD9E8D57)
_PHILOX_W0 = 0x9E3779B9
_PHILOX_W1 = 0xBB67AE85


def philox4x32(c0, c1, c2, c3, k0, k1, rounds=10):
    """Philox4x32 block function on broadcastable uint32 arrays.

    Returns four uint32 arrays.  Round function and key schedule as published
    (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
    SC'11; Random123 philox.h)."""
    c0, c1, c2, c3 = np.broadcast_arrays(
        np.asarray(c0, dtype=U64), np.asarray(c1, dtype=U64), np.asarray(c2, dtype=U64), np.asarray(c3, dtype=U64)
    )
    k0 = int(k0) & MASK32
    k1 = int(k1) & MASK32
    m32 = U64(MASK32)
    s32 = U64(32)
    for _ in range(rounds):
        p0 = _PHILOX_M0 * c0
        p1 = _PHILOX_M1 * c2
        hi0, lo0 = p0 >> s32, p0 & m32
        hi1, lo1 = p1 >> s32, p1 & m32
        c0, c1, c2, c3 = (hi1 ^ c1 ^ U64(k0)), lo1, (hi0 ^ c3 ^ U64(k1)), lo0
        k0 = (k0 + _PHILOX_W0) & MASK32
        k1 = (k1 + _PHILOX_W1) & MASK32
    return c0.astype(U32), c1.astype(U32), c2.astype(U32), c3.astype(U32)


def _key(seed):
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    return seed & MASK32, seed >> 32


def _c3(tag, bank=0, class_id=0):
    return tag | (bank << 8) | (np.asarray(class_id, dtype=np.int64) << 16)


# --------------------------------------------------------------------------
# K11 / K12: initialisation (kernels.py:622-664)
# --------------------------------------------------------------------------


def _fresh_bank(clauses, chunks, state_bits):
    """State 2**(B-1) - 1 for every automaton: low planes all ones, top plane
    zero (kernels.py:655-660, 629-634)."""
    bank = np.full((clauses, chunks, state_bits), MASK32, dtype=U32)
    bank[:, :, state_bits - 1] = 0
    return bank


def prepare(cfg, seed, step=0):
    """kernels.py:638-664.  Returns ``(ta_state, clause_weights)``.

    Weights are random +-1 when NEGATIVE_CLAUSES == 1 (``1 - 2*(draw % 2)``,
    kernels.py:647-648), else 1."""
    ta_state = _fresh_bank(cfg.clauses, cfg.la_chunks, cfg.state_bits)
    if cfg.negative_clauses == 1:
        k0, k1 = _key(seed)
        clause = np.arange(cfg.clauses).reshape(1, -1)
        class_id = np.arange(cfg.classes).reshape(-1, 1)
        r0, _, _, _ = philox4x32(clause, class_id, int(step) & MASK32, TAG_PREPARE, k0, k1)
        weights = (1 - 2 * (r0 & U32(1)).astype(np.int32)).astype(np.int32)
    else:
        weights = np.ones((cfg.classes, cfg.clauses), dtype=np.int32)
    return ta_state, weights


def prepare_message_ta_state(cfg):
    """kernels.py:622-636."""
    return _fresh_bank(cfg.clauses, cfg.message_chunks, cfg.state_bits)


# --------------------------------------------------------------------------
# K1 / K2: clause evaluation per node (kernels.py:407-530)
# --------------------------------------------------------------------------


def _include_plane(bank, state_bits, tail_filter):
    inc = bank[:, :, state_bits - 1].copy()
    inc[:, -1] &= U32(tail_filter)
    return inc


def _popcount32(a):
    a = a.astype(U32)
    a = a - ((a >> U32(1)) & U32(0x55555555))
    a = (a & U32(0x33333333)) + ((a >> U32(2)) & U32(0x33333333))
    a = (a + (a >> U32(4))) & U32(0x0F0F0F0F)
    return ((a * U32(0x01010101)) >> U32(24)).astype(np.int32)


def _node_filter(number_of_nodes):
    r = number_of_nodes % 32
    return MASK32 if r == 0 else (~(MASK32 << r)) & MASK32


def _clause_node_bits(inc, rows, tail_filter, node_type, number_of_node_types, clauses, node_chunks, number_of_nodes):
    """Truth of every clause at every node, packed into node-chunk words the
    way kernels.py:443-466 leaves them: chunks past the graph's last chunk are
    0xFFFFFFFF (never read by any consumer), the last valid chunk is masked."""
    rows = rows.copy()
    rows[:, -1] &= U32(tail_filter)
    # violated[c][n] = some included literal is 0 at node n
    violated = np.empty((clauses, rows.shape[0]), dtype=bool)
    block = max(1, (1 << 24) // max(1, rows.shape[0] * rows.shape[1]))
    not_rows = ~rows
    for c0 in range(0, clauses, block):
        violated[c0 : c0 + block] = ((inc[c0 : c0 + block, None, :] & not_rows[None, :, :]) != 0).any(axis=2)
    type_ok = node_type[None, :].astype(np.int64) == (np.arange(clauses) % number_of_node_types)[:, None]
    truth = (~violated) & type_ok
    out = np.full((clauses, node_chunks), MASK32, dtype=U32)
    n_chunks = (number_of_nodes - 1) // 32 + 1
    padded = np.zeros((clauses, n_chunks * 32), dtype=np.uint8)
    padded[:, :number_of_nodes] = truth
    # positions past number_of_nodes inside the last chunk: the reference's
    # loop leaves them 1 and then applies node_filter; both give 0.
    out[:, :n_chunks] = np.packbits(padded, axis=1, bitorder="little").view("<u4")
    return out


def calculate_messages(cfg, ta_state, node_type, number_of_node_types, number_of_nodes, X_rows):
    """kernels.py:407-468 for one graph.

    ``node_type`` and ``X_rows`` are the graph's slices (the reference offsets
    both by ``graph_index``).  Returns ``(bitmap, number_of_include_actions)``."""
    inc = _include_plane(ta_state, cfg.state_bits, cfg.filter)
    n_incl = _popcount32(inc).sum(axis=1).astype(np.int32)  # kernels.py:266-277
    bitmap = _clause_node_bits(
        inc, np.asarray(X_rows, dtype=U32), cfg.filter, node_type, number_of_node_types,
        cfg.clauses, cfg.node_chunks, number_of_nodes,
    )
    return bitmap, n_incl


def calculate_messages_conditional(
    cfg, message_ta_state, node_type, number_of_node_types, number_of_nodes, condition, n_incl, clause_X
):
    """kernels.py:470-530.  ``condition`` is the previous layer's bitmap;
    returns ``(bitmap, n_incl + message includes)``."""
    inc = _include_plane(message_ta_state, cfg.state_bits, cfg.message_filter)
    n_incl = (n_incl + _popcount32(inc).sum(axis=1)).astype(np.int32)  # kernels.py:501-503
    own = _clause_node_bits(
        inc, np.asarray(clause_X, dtype=U32)[:number_of_nodes], cfg.message_filter, node_type,
        number_of_node_types, cfg.clauses, cfg.node_chunks, number_of_nodes,
    )
    return condition & own, n_incl


# --------------------------------------------------------------------------
# K3 / K4 / K5: message construction (kernels.py:532-615)
# --------------------------------------------------------------------------


def _unpack_bitmap(bitmap, number_of_nodes):
    """bool [CLAUSES][number_of_nodes]."""
    n_chunks = (number_of_nodes - 1) // 32 + 1
    bits = np.unpackbits(np.ascontiguousarray(bitmap[:, :n_chunks]).view(np.uint8), axis=1, bitorder="little")
    return bits[:, :number_of_nodes].astype(bool)


def prepare_messages(cfg, number_of_nodes):
    """kernels.py:532-547: positive half 0, negated half 1, one int per literal."""
    x_int = np.zeros((number_of_nodes, cfg.message_literals), dtype=U32)
    x_int[:, cfg.message_size:] = 1
    return x_int


def exchange_messages(cfg, number_of_nodes, hypervectors, bitmap, n_edges, edge, x_int):
    """kernels.py:549-590.  ``n_edges`` and ``edge`` are the graph's slices:
    out-edge counts per node and the contiguous ``(destination, type)`` rows."""
    truth = _unpack_bitmap(bitmap, number_of_nodes)  # [C][N]
    n_edges = np.asarray(n_edges, dtype=np.int64)[:number_of_nodes]
    total = int(n_edges.sum())
    if total == 0:
        return x_int
    edge = np.asarray(edge, dtype=np.int64).reshape(-1, 2)[:total]
    src = np.repeat(np.arange(number_of_nodes), n_edges)
    clause_idx, edge_idx = np.nonzero(truth[:, src])
    hv = np.asarray(hypervectors, dtype=np.int64).reshape(cfg.clauses, cfg.message_bits)
    for j in range(cfg.message_bits):
        shifted = (hv[clause_idx, j] + edge[edge_idx, 1]) % cfg.message_size  # kernels.py:581
        x_int[edge[edge_idx, 0], shifted] = 1
        x_int[edge[edge_idx, 0], cfg.message_size + shifted] = 0
    return x_int


def encode_messages(cfg, number_of_nodes, x_int):
    """kernels.py:592-615: pack 32 literals per word, zero padding."""
    bits = np.zeros((number_of_nodes, cfg.message_chunks * 32), dtype=np.uint8)
    bits[:, : cfg.message_literals] = x_int != 0
    return np.ascontiguousarray(np.packbits(bits, axis=1, bitorder="little").view("<u4")).astype(U32)


def build_messages(cfg, number_of_nodes, hypervectors, bitmap, n_edges, edge):
    """K3 -> K4 -> K5 as the driver chains them (tm.py:598-630)."""
    x_int = prepare_messages(cfg, number_of_nodes)
    x_int = exchange_messages(cfg, number_of_nodes, hypervectors, bitmap, n_edges, edge, x_int)
    return encode_messages(cfg, number_of_nodes, x_int)


# --------------------------------------------------------------------------
# K6: class sums (kernels.py:279-317)
# --------------------------------------------------------------------------


def clause_outputs(cfg, bitmap, number_of_nodes):
    """1 where the clause is true at some node (kernels.py:297-308)."""
    # C division: an empty graph still reads one (unmasked) chunk, kernels.py:289-295
    n_chunks = 1 if number_of_nodes == 0 else (number_of_nodes - 1) // 32 + 1
    words = bitmap[:, :n_chunks].copy()
    words[:, -1] &= U32(_node_filter(number_of_nodes))
    return (words != 0).any(axis=1)


def evaluate(cfg, bitmap, clause_weights, number_of_nodes):
    """kernels.py:279-317: unclipped weighted vote per class, int32."""
    fired = clause_outputs(cfg, bitmap, number_of_nodes)
    w = np.asarray(clause_weights, dtype=np.int64).reshape(cfg.classes, cfg.clauses)
    return (w[:, fired].sum(axis=1)).astype(np.int32)


# --------------------------------------------------------------------------
# K7: pick one true node per clause (kernels.py:319-354)
# --------------------------------------------------------------------------


def select_clause_node(cfg, seed, step, bitmap, number_of_nodes):
    """Uniform choice among the nodes where the clause is true, -1 if none.

    The reference takes ``list[curand % len]``; here the index is
    ``(r * len) >> 32`` with ``r`` the first Philox word at counter
    ``(clause, 0, step, TAG_CLAUSE_NODE)``."""
    if number_of_nodes == 0:
        return np.full(cfg.clauses, -1, dtype=np.int32)
    truth = _unpack_bitmap(bitmap, number_of_nodes)
    count = truth.sum(axis=1).astype(np.int64)
    k0, k1 = _key(seed)
    r0, _, _, _ = philox4x32(np.arange(cfg.clauses), 0, int(step) & MASK32, TAG_CLAUSE_NODE, k0, k1)
    pick = (r0.astype(np.int64) * count) >> 32
    rank = np.cumsum(truth, axis=1) - 1  # rank of each true node
    chosen = truth & (rank == pick[:, None])
    node = np.where(count > 0, chosen.argmax(axis=1), -1)
    return node.astype(np.int32)


# --------------------------------------------------------------------------
# K8: feedback decision and weight update (kernels.py:356-405)
# --------------------------------------------------------------------------


def select_clause_updates(cfg, seed, step, clause_weights, class_sum, y_row, clause_node):
    """Returns ``class_clause_update [CLASSES][CLAUSES]`` and updates
    ``clause_weights`` in place.  ``y_row`` is ``encoded_Y[example]``.

    Draws: counter ``(clause, class, step, TAG_CLAUSE_UPDATES)``; word 0 gates
    negative targets (keep when ``r0 < q_threshold``), word 1 gates on the
    prediction error (keep when ``r1 * 2T < err * 2**32``), standing for
    kernels.py:384."""
    T = cfg.threshold
    w = clause_weights.reshape(cfg.classes, cfg.clauses)
    cs = np.clip(np.asarray(class_sum, dtype=np.int64), -T, T)[:, None]  # kernels.py:373-378
    y = np.asarray(y_row, dtype=np.int64)[:, None]
    target = 1 - 2 * (cs > y).astype(np.int64)
    sign = np.where(w >= 0, 1, -1).astype(np.int64)
    err = np.abs(y - cs)
    k0, k1 = _key(seed)
    clause = np.arange(cfg.clauses).reshape(1, -1)
    class_id = np.arange(cfg.classes).reshape(-1, 1)
    r0, r1, _, _ = philox4x32(clause, class_id, int(step) & MASK32, TAG_CLAUSE_UPDATES, k0, k1)
    skip_q = (target == -1) & (r0.astype(np.int64) >= q_threshold(cfg.q, cfg.classes))
    skip_err = r1.astype(np.int64) * (2 * T) >= (err << 32)
    skip = skip_q | skip_err
    update = np.where(skip, 0, target * sign).astype(np.int32)
    fired = (np.asarray(clause_node) != -1)[None, :]
    w64 = w.astype(np.int64)
    grow = (update > 0) & fired & (np.abs(w64) < INT_MAX)  # kernels.py:389-390
    shrink = (update < 0) & fired  # kernels.py:391-392
    w64 = w64 + np.where(grow, sign, 0) - np.where(shrink, sign, 0)
    if cfg.negative_clauses == 0:  # kernels.py:394-398
        w64 = np.where(shrink & (w64 < 1), 1, w64)
    w[:, :] = w64.astype(np.int32)
    return update


# --------------------------------------------------------------------------
# K9 / K10: Type I / II feedback (kernels.py:55-242)
# --------------------------------------------------------------------------


def inc(bank, active):
    """kernels.py:55-74 on every (clause, chunk) at once: saturating +1 on the
    automata flagged in ``active`` (ripple carry, residual carry saturates)."""
    carry = active.astype(U32)
    for b in range(bank.shape[2]):
        nxt = bank[:, :, b] & carry
        bank[:, :, b] ^= carry
        carry = nxt
    for b in range(bank.shape[2]):
        bank[:, :, b] |= carry


def dec(bank, active):
    """kernels.py:77-96: saturating -1."""
    carry = active.astype(U32)
    for b in range(bank.shape[2]):
        nxt = ~bank[:, :, b] & carry
        bank[:, :, b] ^= carry
        carry = nxt
    for b in range(bank.shape[2]):
        bank[:, :, b] &= ~carry


def feedback_bits(seed, step, bank_id, class_id, clauses, chunks, threshold16):
    """32 Bernoulli bits per (clause, word): stands for the 32
    ``curand_uniform <= 1/s`` draws of kernels.py:113-118, 157-162.

    Word ``w`` of clause ``c`` uses four Philox blocks at counters
    ``(c, 4*w + j, step, TAG_FEEDBACK | bank << 8 | class << 16)``, j = 0..3;
    bit ``b`` takes block ``b // 8``, output word ``(b % 8) // 2``, low half for
    even ``b`` and high half for odd ``b``, and is set when that 16-bit value
    is below ``threshold16``."""
    k0, k1 = _key(seed)
    clause = np.arange(clauses).reshape(-1, 1, 1)
    sub = (np.arange(chunks).reshape(1, -1, 1) * 4) + np.arange(4).reshape(1, 1, -1)
    out = philox4x32(clause, sub, int(step) & MASK32, int(_c3(TAG_FEEDBACK, bank_id, class_id)), k0, k1)
    words = np.stack(out, axis=-1).astype(np.int64)  # [C][chunks][4 blocks][4 words]
    halves = np.stack([words & 0xFFFF, words >> 16], axis=-1)  # [...][4][4][2]
    below = (halves.reshape(clauses, chunks, 32) < threshold16).astype(np.uint64)
    return (below << np.arange(32, dtype=np.uint64)).sum(axis=2).astype(U32)


def _feedback(cfg, seed, step, bank_id, s, bank, clause_node, n_incl, literal_rows, class_clause_update):
    """Shared body of ``update`` and ``update_message``
    (kernels.py:98-183, 185-242): classes are applied in ascending order to the
    same bank (kernels.py:205-207, 236-238)."""
    clauses, chunks, _ = bank.shape
    clause_node = np.asarray(clause_node, dtype=np.int64)
    fired = clause_node != -1
    within = np.asarray(n_incl, dtype=np.int64) <= cfg.max_included_literals
    x = np.zeros((clauses, chunks), dtype=U32)
    x[fired] = np.asarray(literal_rows, dtype=U32)[clause_node[fired]]
    thr = feedback_threshold(s)
    top = cfg.state_bits - 1
    for class_id in range(cfg.classes):
        sign = np.asarray(class_clause_update[class_id], dtype=np.int64)
        type1 = sign > 0
        type2 = (sign < 0) & fired
        if type1.any():
            fb = feedback_bits(seed, step, bank_id, class_id, clauses, chunks, thr)
            reinforce = (type1 & fired & within)[:, None]
            weaken = (type1 & ~(fired & within))[:, None]
            if cfg.boost_true_positive_feedback == 1:
                inc(bank, np.where(reinforce, x, 0))
            else:
                inc(bank, np.where(reinforce, x & ~fb, 0))
            dec(bank, np.where(reinforce, ~x & fb, 0))
            dec(bank, np.where(weaken, fb, 0))
        if type2.any():
            inc(bank, np.where(type2[:, None], ~x & ~bank[:, :, top], 0))


def update(cfg, seed, step, s, ta_state, clause_node, n_incl, X_rows, class_clause_update):
    """kernels.py:213-242 (layer-0 bank, literals of the selected node)."""
    _feedback(cfg, seed, step, 0, s, ta_state, clause_node, n_incl, X_rows, class_clause_update)


def update_message(cfg, seed, step, bank_id, s, message_ta_state, clause_node, n_incl, clause_X, class_clause_update):
    """kernels.py:185-211 (message bank ``bank_id`` >= 1, literals = the packed
    messages of the selected node)."""
    _feedback(cfg, seed, step, bank_id, s, message_ta_state, clause_node, n_incl, clause_X, class_clause_update)


# --------------------------------------------------------------------------
# drivers: tm.py:563-812
# --------------------------------------------------------------------------


@dataclass
class Model:
    """Device state of the reference (tm.py:110-124) held on the host."""

    cfg: Config
    depth: int
    s: tuple
    ta_state: np.ndarray
    message_ta_state: list
    clause_weights: np.ndarray
    hypervectors: np.ndarray
    seed: int = 0
    step: int = 0


def new_model(cfg, depth, s, hypervectors, seed):
    ta_state, weights = prepare(cfg, seed, 0)
    banks = [prepare_message_ta_state(cfg) for _ in range(depth - 1)]
    s = tuple(s) if isinstance(s, (tuple, list)) else (s,) * depth
    return Model(cfg, depth, s, ta_state, banks, weights, np.asarray(hypervectors, dtype=U32), seed, 0)


def evaluate_graph(model, graphs, e):
    """tm.py:563-662 for graph ``e``: returns
    ``(final bitmap, class_sum, n_incl, [clause_X per message layer])``."""
    cfg = model.cfg
    n = int(graphs.number_of_graph_nodes[e])
    base = int(graphs.node_index[e])
    node_type = graphs.node_type[base : base + n]
    rows = graphs.X[base : base + n]
    n_types = graphs.number_of_node_types()
    bitmap, n_incl = calculate_messages(cfg, model.ta_state, node_type, n_types, n, rows)
    layers = []
    if model.depth > 1:
        n_edges = graphs.number_of_graph_node_edges[base : base + n]
        e0 = int(graphs.edge_index[base]) if n > 0 else 0  # a trailing graph without nodes has no entry
        edge = graphs.edge[e0 : e0 + int(n_edges.astype(np.int64).sum())]
    for d in range(model.depth - 1):
        clause_X = build_messages(cfg, n, model.hypervectors, bitmap, n_edges, edge)
        layers.append(clause_X)
        bitmap, n_incl = calculate_messages_conditional(
            cfg, model.message_ta_state[d], node_type, n_types, n, bitmap, n_incl, clause_X
        )
    class_sum = evaluate(cfg, bitmap, model.clause_weights, n)
    return bitmap, class_sum, n_incl, layers


def score(model, graphs, indices=None):
    """tm.py:786-812."""
    if indices is None:
        indices = range(graphs.number_of_graphs)
    out = np.zeros((len(indices), model.cfg.classes), dtype=np.int32)
    for i, e in enumerate(indices):
        out[i] = evaluate_graph(model, graphs, e)[1]
    return out


def transform(model, graphs, indices=None, nodewise=False):
    """tm.py:814-900 with kernels.py:671-710: per graph, 1 where the clause is true
    at some node of the graph (``nodewise``: its truth at every node, zero-padded
    to the largest graph), next to the class sums.  Unlike `evaluate`, the
    transform kernels loop over the graph's nodes, so a graph without nodes
    gives zeros."""
    cfg = model.cfg
    if indices is None:
        indices = range(graphs.number_of_graphs)
    width = int(graphs.number_of_graph_nodes.max()) if graphs.number_of_graphs else 0
    shape = (len(indices), cfg.clauses, width) if nodewise else (len(indices), cfg.clauses)
    out = np.zeros(shape, dtype=np.int32)
    sums = np.zeros((len(indices), cfg.classes), dtype=np.int32)
    for i, e in enumerate(indices):
        n = int(graphs.number_of_graph_nodes[e])
        bitmap, sums[i], _, _ = evaluate_graph(model, graphs, e)
        if n == 0:
            continue
        truth = _unpack_bitmap(bitmap, n)
        if nodewise:
            out[i, :, :n] = truth
        else:
            out[i] = truth.any(axis=1)
    return out, sums


def get_ta_states(bank, state_bits, literals):
    """kernels.py:718-757: the integer state of every automaton, uint32 [CLAUSES][literals]."""
    bank = np.asarray(bank, dtype=U32)
    clauses, chunks, _ = bank.shape
    out = np.zeros((clauses, chunks * 32), dtype=U32)
    for b in range(state_bits):
        plane = np.unpackbits(np.ascontiguousarray(bank[:, :, b]).view(np.uint8), axis=1, bitorder="little")
        out |= plane.astype(U32) << U32(b)
    return out[:, :literals]


def get_hyperliterals(bank, state_bits, literals):
    """kernels.py:761-790: 1 where the automaton's action is include, uint32 [CLAUSES][literals]."""
    bank = np.asarray(bank, dtype=U32)
    plane = np.unpackbits(np.ascontiguousarray(bank[:, :, state_bits - 1]).view(np.uint8), axis=1, bitorder="little")
    return plane[:, :literals].astype(U32)


def fit_graph(model, graphs, encoded_Y, e):
    """One iteration of the loop at tm.py:669-747."""
    cfg = model.cfg
    n = int(graphs.number_of_graph_nodes[e])
    base = int(graphs.node_index[e])
    bitmap, class_sum, n_incl, layers = evaluate_graph(model, graphs, e)
    clause_node = select_clause_node(cfg, model.seed, model.step, bitmap, n)
    updates = select_clause_updates(
        cfg, model.seed, model.step, model.clause_weights, class_sum, encoded_Y[e], clause_node
    )
    update(cfg, model.seed, model.step, model.s[0], model.ta_state, clause_node, n_incl,
           graphs.X[base : base + n], updates)
    for d in range(model.depth - 1):
        update_message(cfg, model.seed, model.step, d + 1, model.s[d + 1], model.message_ta_state[d],
                       clause_node, n_incl, layers[d], updates)
    model.step += 1
    return bitmap, class_sum, clause_node, updates


def fit(model, graphs, encoded_Y, epochs=1, indices=None):
    """tm.py:664-752 (the two nested loops)."""
    if indices is None:
        indices = range(graphs.number_of_graphs)
    for _ in range(epochs):
        for e in indices:
            fit_graph(model, graphs, encoded_Y, e)


def encode_labels(Y, classes, T):
    """tm.py:949-951."""
    Y = np.asarray(Y)
    out = np.full((Y.shape[0], classes), -T, dtype=np.int32)
    out[np.arange(Y.shape[0]), Y.astype(np.int64)] = T
    return out
