"""Clause evaluation, messages and class sums of the oracle against brute-force
literal-level / set-level restatements written independently in pure Python."""

import numpy as np
import pytest

from oracle import gtm_oracle as o
from tests import helpers


def bit(words, k):
    return (int(words[k // 32]) >> (k % 32)) & 1


def brute_clause_truth(cfg, bank, chunks, n_literals, rows, node_type, n_types):
    """truth[c][n] = node type matches and every included literal is 1."""
    top = cfg.state_bits - 1
    out = np.zeros((cfg.clauses, len(rows)), dtype=bool)
    for c in range(cfg.clauses):
        included = [k for k in range(n_literals) if bit(bank[c, :, top], k)]
        for n, row in enumerate(rows):
            out[c, n] = int(node_type[n]) == c % n_types and all(bit(row, k) for k in included)
    return out


def pack_truth(cfg, truth, n):
    words = np.full((cfg.clauses, cfg.node_chunks), 0xFFFFFFFF, dtype=np.uint32)
    for c in range(cfg.clauses):
        for ch in range((n - 1) // 32 + 1):
            v = 0
            for p in range(32):
                if ch * 32 + p < n and truth[c, ch * 32 + p]:
                    v |= 1 << p
            words[c, ch] = v
    return words


CASES = [
    dict(seed=5, g=dict(n_graphs=3, max_nodes=45, hv_size=20), clauses=12, density=0.04),       # 40 literals: tail filter
    dict(seed=6, g=dict(n_graphs=3, max_nodes=64, hv_size=16, min_nodes=64, node_types=("a", "b", "c")), clauses=10, density=0.02),
    dict(seed=7, g=dict(n_graphs=4, max_nodes=5, hv_size=40), clauses=9, density=0.3),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "seed%d" % c["seed"])
def test_calculate_messages_is_literal_level_and(case):
    graphs = helpers.random_graphs(case["seed"], **case["g"])
    cfg = helpers.oracle_config(graphs, classes=2, clauses=case["clauses"])
    model = helpers.random_model(case["seed"], cfg, 1, include_density=case["density"])
    top = cfg.state_bits - 1
    model.ta_state[0, :, top] = 0                      # an empty clause
    model.ta_state[1, :, top] = 0
    model.ta_state[1, 0, top] = 1 | (1 << (graphs.hypervector_size % 32)) if graphs.hypervector_size < 32 else 1
    for e in range(graphs.number_of_graphs):
        n, base = int(graphs.number_of_graph_nodes[e]), int(graphs.node_index[e])
        rows, types = graphs.X[base:base + n], graphs.node_type[base:base + n]
        got, n_incl = o.calculate_messages(cfg, model.ta_state, types, graphs.number_of_node_types(), n, rows)
        truth = brute_clause_truth(cfg, model.ta_state, cfg.la_chunks, cfg.literals, rows, types,
                                   graphs.number_of_node_types())
        assert np.array_equal(got, pack_truth(cfg, truth, n))
        # the empty clause is true on every node of its type (kernels.py:443-456)
        assert np.array_equal(truth[0], types == 0)
        want_incl = [sum(bit(model.ta_state[c, :, top], k) for k in range(cfg.literals)) for c in range(cfg.clauses)]
        assert list(n_incl) == want_incl


def test_literal_and_its_negation_never_both_hold():
    graphs = helpers.random_graphs(8, n_graphs=2, max_nodes=30, hv_size=16)
    cfg = helpers.oracle_config(graphs, classes=2, clauses=3)
    model = helpers.random_model(8, cfg, 1, include_density=0.0)
    model.ta_state[:, :, cfg.state_bits - 1] = 0
    model.ta_state[1, 0, cfg.state_bits - 1] = (1 << 3) | (1 << (3 + 16))  # x3 AND NOT x3
    n = int(graphs.number_of_graph_nodes[0])
    got, _ = o.calculate_messages(cfg, model.ta_state, graphs.node_type[:n], 1, n, graphs.X[:n])
    assert not o._unpack_bitmap(got, n)[1].any()
    assert o._unpack_bitmap(got, n)[0].all()


def test_padding_includes_are_ignored():
    graphs = helpers.random_graphs(9, n_graphs=1, max_nodes=10, hv_size=20)  # literals = 40, 24 padding bits
    cfg = helpers.oracle_config(graphs, classes=2, clauses=2)
    model = helpers.random_model(9, cfg, 1, include_density=0.0)
    top = cfg.state_bits - 1
    model.ta_state[:, :, top] = 0
    model.ta_state[0, 1, top] = 0xFFFFFF00  # only padding positions of the last word
    n = int(graphs.number_of_graph_nodes[0])
    got, n_incl = o.calculate_messages(cfg, model.ta_state, graphs.node_type[:n], 1, n, graphs.X[:n])
    assert o._unpack_bitmap(got, n)[0].all() and n_incl[0] == 0


def brute_messages(cfg, n, hv, truth, n_edges, edge):
    """Set semantics: a node's positive message bits are the union, over its
    incoming edges (src -> node, type) and the clauses true at src, of
    (h + type) mod M; the negated half is the complement."""
    pos = [set() for _ in range(n)]
    at = 0
    for src in range(n):
        for _ in range(int(n_edges[src])):
            dst, kind = int(edge[at][0]), int(edge[at][1])
            at += 1
            for c in range(cfg.clauses):
                if truth[c, src]:
                    for h in hv[c]:
                        pos[dst].add((int(h) + kind) % cfg.message_size)
    out = np.zeros((n, cfg.message_chunks), dtype=np.uint32)
    for node in range(n):
        for k in range(cfg.message_size):
            lit = k if k in pos[node] else k + cfg.message_size
            out[node, lit // 32] |= np.uint32(1 << (lit % 32))
    return out


@pytest.mark.parametrize("message_size,message_bits", [(37, 2), (16, 1), (64, 3)])
def test_messages_are_rotated_unions(message_size, message_bits):
    graphs = helpers.random_graphs(13, n_graphs=4, max_nodes=40, hv_size=16, edge_types=("a", "b", "c", "d", "e"),
                                   max_degree=4)
    cfg = helpers.oracle_config(graphs, classes=2, clauses=11, depth=2, message_size=message_size,
                                message_bits=message_bits)
    model = helpers.random_model(13, cfg, 2, include_density=0.03)
    model.hypervectors[0, 0] = message_size - 1  # rotation wraps around for edge types >= 1
    for e in range(graphs.number_of_graphs):
        n, base = int(graphs.number_of_graph_nodes[e]), int(graphs.node_index[e])
        n_edges = graphs.number_of_graph_node_edges[base:base + n]
        e0 = int(graphs.edge_index[base])
        edge = graphs.edge[e0:e0 + int(n_edges.sum())]
        bitmap, n_incl = o.calculate_messages(cfg, model.ta_state, graphs.node_type[base:base + n], 1, n,
                                              graphs.X[base:base + n])
        truth = o._unpack_bitmap(bitmap, n)
        got = o.build_messages(cfg, n, model.hypervectors, bitmap, n_edges, edge)
        assert np.array_equal(got, brute_messages(cfg, n, model.hypervectors, truth, n_edges, edge))
        # layer 2 = layer-1 truth AND message clause truth
        nxt, n2 = o.calculate_messages_conditional(cfg, model.message_ta_state[0], graphs.node_type[base:base + n], 1,
                                                   n, bitmap, n_incl, got)
        own = brute_clause_truth(cfg, model.message_ta_state[0], cfg.message_chunks, cfg.message_literals, got,
                                 graphs.node_type[base:base + n], 1)
        assert np.array_equal(o._unpack_bitmap(nxt, n), truth & own)
        top = cfg.state_bits - 1
        extra = [sum(bit(model.message_ta_state[0][c, :, top], k) for k in range(cfg.message_literals))
                 for c in range(cfg.clauses)]
        assert list(n2 - n_incl) == extra


def test_no_edges_gives_blank_messages():
    graphs = helpers.random_graphs(14, n_graphs=1, max_nodes=6, max_degree=0)
    cfg = helpers.oracle_config(graphs, classes=2, clauses=4, depth=2, message_size=20)
    model = helpers.random_model(14, cfg, 2, include_density=0.0)
    n = int(graphs.number_of_graph_nodes[0])
    bitmap, _ = o.calculate_messages(cfg, model.ta_state, graphs.node_type[:n], 1, n, graphs.X[:n])
    got = o.build_messages(cfg, n, model.hypervectors, bitmap, graphs.number_of_graph_node_edges[:n], graphs.edge)
    for row in got:
        assert [bit(row, k) for k in range(64)] == [0] * 20 + [1] * 20 + [0] * 24


def test_class_sums_are_weights_times_clause_outputs():
    graphs = helpers.random_graphs(15, n_graphs=5, max_nodes=70, hv_size=16)
    cfg = helpers.oracle_config(graphs, classes=4, clauses=40)
    model = helpers.random_model(15, cfg, 1, include_density=0.05)
    for e in range(5):
        n, base = int(graphs.number_of_graph_nodes[e]), int(graphs.node_index[e])
        bitmap, _ = o.calculate_messages(cfg, model.ta_state, graphs.node_type[base:base + n], 1, n,
                                         graphs.X[base:base + n])
        fired = o._unpack_bitmap(bitmap, n).any(axis=1)
        want = model.clause_weights.astype(np.int64) @ fired.astype(np.int64)
        assert np.array_equal(o.evaluate(cfg, bitmap, model.clause_weights, n), want)
        assert np.array_equal(o.evaluate_graph(model, graphs, e)[1], want)


def test_fresh_model_votes_with_all_its_weights():
    """Empty clauses fire: a freshly initialised model scores sum_c W[k][c]."""
    graphs = helpers.random_graphs(16, n_graphs=2, max_nodes=9)
    cfg = helpers.oracle_config(graphs, classes=3, clauses=25, depth=2)
    model = o.new_model(cfg, 2, 1.0, np.zeros((25, 2), dtype=np.uint32) + [[0, 1]], seed=4)
    assert np.array_equal(o.score(model, graphs), np.tile(model.clause_weights.sum(axis=1), (2, 1)))
