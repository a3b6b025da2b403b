"""Pins for the oracle's read-outs (transform, automaton states, include actions):
closed forms and brute force that do not restate the oracle's own formulas."""

import numpy as np

from oracle import gtm_oracle as o
from tests import helpers


def encode_states(states, state_bits):
    """Integer states [C][literals] -> bit-sliced bank [C][chunks][state_bits], built bit by bit."""
    clauses, literals = states.shape
    chunks = (literals - 1) // 32 + 1
    bank = np.zeros((clauses, chunks, state_bits), dtype=np.uint32)
    for c in range(clauses):
        for k in range(literals):
            for b in range(state_bits):
                if (int(states[c, k]) >> b) & 1:
                    bank[c, k // 32, b] |= np.uint32(1 << (k % 32))
    return bank


def test_ta_states_and_actions_decode_known_integers():
    rng = np.random.default_rng(3)
    for state_bits, literals in [(8, 40), (4, 64), (10, 7), (1, 33)]:
        states = rng.integers(0, 2 ** state_bits, size=(5, literals))
        bank = encode_states(states, state_bits)
        assert np.array_equal(o.get_ta_states(bank, state_bits, literals), states)
        # include = state in the upper half
        assert np.array_equal(o.get_hyperliterals(bank, state_bits, literals), states >= 2 ** (state_bits - 1))


def test_fresh_bank_is_one_below_include():
    cfg = o.Config(classes=2, clauses=3, literals=40, state_bits=8, threshold=10, q=1.0, max_included_literals=None,
                   max_nodes=4, message_size=16, message_bits=1)
    ta, _ = o.prepare(cfg, 1)
    assert (o.get_ta_states(ta, 8, 40) == 127).all() and not o.get_hyperliterals(ta, 8, 40).any()


def test_transform_is_clause_truth_by_brute_force():
    """transform == for every clause, whether some node of its type carries all its included literals
    (layer 0; literal-level Python loops), and the nodewise form is that truth per node."""
    graphs = helpers.random_graphs(5, n_graphs=5, hv_size=12, node_types=("a", "b"), sizes=[4, 0, 33, 1, 7])
    cfg = helpers.oracle_config(graphs, classes=3, clauses=12)
    model = helpers.random_model(5, cfg, 1, include_density=0.08)
    got, sums = o.transform(model, graphs)
    wide, sums_wide = o.transform(model, graphs, nodewise=True)
    assert wide.shape == (5, 12, 33) and np.array_equal(sums, sums_wide) and np.array_equal(sums, o.score(model, graphs))
    included = o.get_hyperliterals(model.ta_state, cfg.state_bits, cfg.literals)
    for e in range(5):
        n, base = int(graphs.number_of_graph_nodes[e]), int(graphs.node_index[e])
        for c in range(cfg.clauses):
            truth = []
            for node in range(n):
                row = graphs.X[base + node]
                ok = int(graphs.node_type[base + node]) == c % 2
                for k in range(cfg.literals):
                    if included[c, k] and not (int(row[k // 32]) >> (k % 32)) & 1:
                        ok = False
                truth.append(int(ok))
            assert list(wide[e, c, :n]) == truth and not wide[e, c, n:].any()
            assert got[e, c] == int(any(truth))
    # a graph without nodes transforms to zeros although it scores as if every clause were true
    assert not got[1].any() and np.array_equal(sums[1], model.clause_weights.sum(axis=1))


def test_transform_follows_the_last_layer():
    graphs = helpers.random_graphs(6, n_graphs=4, max_nodes=20, hv_size=16, edge_types=("x", "y"))
    cfg = helpers.oracle_config(graphs, classes=2, clauses=20, depth=2, message_size=16)
    model = helpers.random_model(6, cfg, 2, include_density=0.03, message_density=0.05)
    got, _ = o.transform(model, graphs)
    for e in range(4):
        bitmap = o.evaluate_graph(model, graphs, e)[0]
        assert np.array_equal(got[e].astype(bool), o.clause_outputs(cfg, bitmap, int(graphs.number_of_graph_nodes[e])))
