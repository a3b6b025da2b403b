"""Shared builders for the tests: random ragged graphs, random model states."""

import numpy as np

from graphtsetlinmachine_amd.graphs import Graphs
from oracle import gtm_oracle as o


def random_graphs(seed, n_graphs=6, max_nodes=40, hv_size=20, hv_bits=2, n_symbols=7, node_types=("Plain",),
                  edge_types=("Plain",), max_degree=3, min_nodes=1, parent=None, sizes=None):
    """Ragged graphs built through the per-call API: several node and edge
    types, self-loops, parallel edges, nodes without out-edges."""
    rng = np.random.default_rng(seed)
    symbols = ["s%d" % i for i in range(n_symbols)]
    if parent is None:
        saved = np.random.get_state()
        np.random.seed(seed)
        g = Graphs(n_graphs, symbols=symbols, hypervector_size=hv_size, hypervector_bits=hv_bits)
        np.random.set_state(saved)
    else:
        g = Graphs(n_graphs, init_with=parent)
    sizes = rng.integers(min_nodes, max_nodes + 1, size=n_graphs) if sizes is None else np.asarray(sizes)
    for i, n in enumerate(sizes):
        g.set_number_of_graph_nodes(i, int(n))
    g.prepare_node_configuration()
    degrees = []
    for i, n in enumerate(sizes):
        deg = rng.integers(0, max_degree + 1, size=n) if max_degree > 0 else np.zeros(n, dtype=int)
        degrees.append(deg)
        for node in range(n):
            g.add_graph_node(i, "n%d" % node, int(deg[node]), str(node_types[rng.integers(len(node_types))]))
    g.prepare_edge_configuration()
    for i, n in enumerate(sizes):
        for node in range(n):
            for _ in range(int(degrees[i][node])):
                dst = int(rng.integers(n))  # may be the node itself
                g.add_graph_node_edge(i, "n%d" % node, "n%d" % dst, str(edge_types[rng.integers(len(edge_types))]))
            for sym in rng.choice(n_symbols, size=rng.integers(0, 4), replace=False):
                g.add_graph_node_property(i, "n%d" % node, symbols[int(sym)])
    g.encode()
    return g


def oracle_config(graphs, classes, clauses, depth=1, message_size=37, message_bits=2, T=50, q=1.0, state_bits=8,
                  boost=1, max_included=None, max_nodes=None):
    return o.Config(
        classes=classes, clauses=clauses, literals=2 * graphs.hypervector_size, state_bits=state_bits,
        boost_true_positive_feedback=boost, threshold=T, q=q, max_included_literals=max_included,
        negative_clauses=1, max_nodes=max(1, int(max_nodes or graphs.max_number_of_graph_nodes)),  # as tm.py sizes a model for a data set without nodes
        message_size=message_size, message_bits=message_bits,
    )


def random_bank(rng, clauses, chunks, state_bits, include_density):
    """Random automaton states whose include bit (top plane) is set with the
    given probability; lower planes uniform.  Padding lanes are random too."""
    bank = rng.integers(0, 2**32, size=(clauses, chunks, state_bits), dtype=np.uint64).astype(np.uint32)
    top = (rng.random((clauses, chunks, 32)) < include_density).astype(np.uint64)
    bank[:, :, state_bits - 1] = (top << np.arange(32, dtype=np.uint64)).sum(axis=2).astype(np.uint32)
    return bank


def random_model(seed, cfg, depth, s=1.0, include_density=0.03, message_density=0.01, weight_range=20):
    rng = np.random.default_rng(seed)
    hv = np.stack([rng.choice(cfg.message_size, size=cfg.message_bits, replace=False) for _ in range(cfg.clauses)])
    model = o.new_model(cfg, depth, s, hv.astype(np.uint32), seed=seed * 7919 + 13)
    model.ta_state = random_bank(rng, cfg.clauses, cfg.la_chunks, cfg.state_bits, include_density)
    model.message_ta_state = [
        random_bank(rng, cfg.clauses, cfg.message_chunks, cfg.state_bits, message_density) for _ in range(depth - 1)
    ]
    model.clause_weights = rng.integers(-weight_range, weight_range + 1, size=(cfg.classes, cfg.clauses)).astype(np.int32)
    return model
