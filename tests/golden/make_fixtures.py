"""Writes tests/golden/frozen_cases.npz: a few small data sets and model states as plain arrays
(inputs) with the class sums before training, the state after one pass of training and the class
sums after it (expected outputs).

The reference ships no fixtures and cannot run where this is built, so the expected outputs are the
NumPy oracle's (oracle/gtm_oracle.py), written only after the independent C restatement
(oracle/gtm_oracle.c) has produced the same ones.  What the file pins is therefore drift: the two
oracles and the HIP path must keep reproducing these numbers from these inputs
(tests/test_golden.py), whatever is changed in any of them later.

    python tests/golden/make_fixtures.py
"""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import gtm_oracle as o  # noqa: E402
from oracle import gtm_oracle_c as oc  # noqa: E402
from tests import helpers  # noqa: E402

CASES = [
    # depth 1, two node types, graphs of 1..40 nodes
    dict(seed=101, g=dict(n_graphs=30, max_nodes=40, hv_size=24, node_types=("a", "b"), max_degree=0),
         m=dict(classes=4, clauses=64, T=25), depth=1, s=(2.7,), density=(0.03, 0.0)),
    # one message layer, three edge types, self-loops and parallel edges
    dict(seed=102, g=dict(n_graphs=24, max_nodes=33, hv_size=16, edge_types=("l", "r", "x"), max_degree=3),
         m=dict(classes=3, clauses=40, T=20, message_size=64, message_bits=2), depth=2, s=(3.1, 1.8),
         density=(0.02, 0.01)),
    # two message layers, 5-bit automata, no boost, a literal budget, a message size that is no multiple
    # of 32, and graphs without nodes
    dict(seed=103, g=dict(n_graphs=21, max_nodes=20, min_nodes=0, hv_size=20, node_types=("a", "b", "c"),
                          edge_types=("l", "r"), max_degree=2),
         m=dict(classes=5, clauses=33, T=15, message_size=37, message_bits=3, state_bits=5, boost=0, max_included=9),
         depth=3, s=(4.0, 2.2, 1.0), density=(0.05, 0.02)),
]

GRAPH_ARRAYS = ("X", "node_type", "number_of_graph_node_edges", "edge", "node_index", "edge_index",
                "number_of_graph_nodes")


def build(case):
    graphs = helpers.random_graphs(case["seed"], **case["g"])
    cfg = helpers.oracle_config(graphs, depth=case["depth"], **case["m"])
    model = helpers.random_model(case["seed"], cfg, case["depth"], s=case["s"], include_density=case["density"][0],
                                 message_density=case["density"][1])
    rng = np.random.default_rng(case["seed"])
    labels = rng.integers(0, cfg.classes, size=graphs.number_of_graphs)
    return graphs, cfg, model, o.encode_labels(labels, cfg.classes, cfg.threshold)


def main():
    assert oc.available() or oc.build(), "the C restatement is needed to cross-check the outputs"
    out = {"n_cases": np.int64(len(CASES))}
    for i, case in enumerate(CASES):
        graphs, cfg, model, Y = build(case)
        p = "c%d_" % i
        for name in GRAPH_ARRAYS:
            out[p + name] = np.ascontiguousarray(getattr(graphs, name))
        out[p + "graph_scalars"] = np.array([graphs.number_of_graphs, graphs.max_number_of_graph_nodes,
                                             graphs.number_of_nodes, graphs.number_of_node_types(),
                                             graphs.hypervector_size], dtype=np.int64)
        out[p + "config"] = np.array([cfg.classes, cfg.clauses, cfg.literals, cfg.state_bits,
                                      cfg.boost_true_positive_feedback, cfg.threshold, cfg.max_included_literals,
                                      cfg.negative_clauses, cfg.max_nodes, cfg.message_size, cfg.message_bits,
                                      model.depth, model.seed], dtype=np.int64)
        out[p + "q"] = np.float64(cfg.q)
        out[p + "s"] = np.array(model.s, dtype=np.float64)
        out[p + "ta_state"] = model.ta_state.copy()
        for l, b in enumerate(model.message_ta_state):
            out[p + "bank%d" % l] = b.copy()
        out[p + "clause_weights"] = model.clause_weights.copy()
        out[p + "hypervectors"] = model.hypervectors.copy()
        out[p + "encoded_Y"] = Y

        # expected outputs: NumPy oracle, cross-checked by the C restatement on a copy
        twin = o.Model(cfg, model.depth, model.s, model.ta_state.copy(), [b.copy() for b in model.message_ta_state],
                       model.clause_weights.copy(), model.hypervectors.copy(), model.seed, 0)
        before = o.score(model, graphs)
        assert np.array_equal(before, oc.score(twin, graphs)), "case %d: class sums differ between the oracles" % i
        o.fit(model, graphs, Y)
        oc.fit(twin, graphs, Y)
        assert np.array_equal(model.ta_state, twin.ta_state) and np.array_equal(model.clause_weights, twin.clause_weights)
        for a, b in zip(model.message_ta_state, twin.message_ta_state):
            assert np.array_equal(a, b)
        after = o.score(model, graphs)
        assert np.array_equal(after, oc.score(twin, graphs))
        out[p + "sums_before"] = before
        out[p + "ta_after"] = model.ta_state
        for l, b in enumerate(model.message_ta_state):
            out[p + "bank%d_after" % l] = b
        out[p + "weights_after"] = model.clause_weights
        out[p + "sums_after"] = after
        changed = int((out[p + "ta_after"] != out[p + "ta_state"]).sum())
        print("case %d: %d graphs, %d nodes, depth %d, %d automaton words changed by training" %
              (i, graphs.number_of_graphs, graphs.number_of_nodes, model.depth, changed))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "frozen_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
