"""The C restatement of the inference path (oracle/gtm_oracle.c) against the NumPy oracle:
two independent readings of the reference's kernels must give the same class sums."""

import numpy as np
import pytest

from oracle import gtm_oracle as o
from oracle import gtm_oracle_c as oc
from tests import helpers

pytestmark = pytest.mark.skipif(not oc.available(), reason="no gcc and no prebuilt oracle/libgtm_oracle_c.so")

SHAPES = [
    dict(seed=1, g=dict(n_graphs=9, max_nodes=40, hv_size=20), m=dict(classes=3, clauses=70, depth=1)),
    dict(seed=2, g=dict(n_graphs=6, max_nodes=70, hv_size=16, node_types=("a", "b"), edge_types=("x", "y", "z")),
         m=dict(classes=2, clauses=33, depth=2, message_size=37)),
    dict(seed=3, g=dict(n_graphs=5, max_nodes=32, hv_size=64, min_nodes=32),
         m=dict(classes=4, clauses=100, depth=3, message_size=64, message_bits=3)),
    dict(seed=4, g=dict(n_graphs=8, max_nodes=3, hv_size=300, hv_bits=3, n_symbols=9),
         m=dict(classes=5, clauses=20, depth=2, message_size=16, message_bits=1, state_bits=4)),
    # graphs without nodes, among others and at the end; single nodes with self-loops
    dict(seed=5, g=dict(n_graphs=7, hv_size=16, sizes=[5, 0, 33, 1, 0, 40, 0]),
         m=dict(classes=3, clauses=20, depth=3, message_size=16, message_bits=1)),
    dict(seed=6, g=dict(n_graphs=30, max_nodes=1, hv_size=40), m=dict(classes=3, clauses=50, depth=2, message_size=8)),
    dict(seed=7, g=dict(n_graphs=4, max_nodes=361, min_nodes=300, hv_size=128, edge_types=("l", "r", "u", "d")),
         m=dict(classes=10, clauses=80, depth=2, message_size=256)),
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "seed%d" % s["seed"])
@pytest.mark.parametrize("density", [0.0, 0.01, 0.05])
@pytest.mark.parametrize("threads", [1, 3])
def test_c_and_numpy_oracles_agree(shape, density, threads):
    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth)
    model = helpers.random_model(shape["seed"], cfg, depth, include_density=density, message_density=density / 2)
    want = o.score(model, graphs)
    assert np.array_equal(oc.score(model, graphs, threads=threads), want)
    some = [graphs.number_of_graphs - 1, 0]
    assert np.array_equal(oc.score(model, graphs, some, threads=threads), want[some])


def test_c_oracle_on_a_model_trained_by_the_numpy_oracle():
    graphs = helpers.random_graphs(11, n_graphs=30, max_nodes=12, hv_size=16, edge_types=("x", "y"))
    cfg = helpers.oracle_config(graphs, classes=3, clauses=40, depth=2, message_size=32, T=20)
    model = helpers.random_model(11, cfg, 2, s=(2.0, 1.5), include_density=0.02)
    rng = np.random.default_rng(11)
    Y = o.encode_labels(rng.integers(0, 3, size=30), 3, cfg.threshold)
    o.fit(model, graphs, Y, epochs=2)
    assert np.array_equal(oc.score(model, graphs), o.score(model, graphs))


@pytest.mark.parametrize("shape", SHAPES[:6], ids=lambda s: "seed%d" % s["seed"])
@pytest.mark.parametrize("boost,max_included,state_bits,negative", [(1, None, 8, 1), (0, 9, 5, 1), (1, None, 12, 0)])
def test_c_and_numpy_oracles_train_alike(shape, boost, max_included, state_bits, negative):
    """Two epochs, the second split into two calls and run on three threads: banks, weights and step."""
    import copy

    g = dict(shape["g"])
    graphs = helpers.random_graphs(shape["seed"], **g)
    m = dict(shape["m"])
    depth = m.pop("depth")
    m.pop("state_bits", None)
    cfg = helpers.oracle_config(graphs, **m, depth=depth, T=30, boost=boost, max_included=max_included,
                                state_bits=state_bits)
    cfg.negative_clauses = negative
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0, 2.0, 1.0)[:depth] if depth > 1 else 3.0,
                                 include_density=0.03, message_density=0.02)
    twin = copy.deepcopy(model)
    rng = np.random.default_rng(shape["seed"])
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    o.fit(model, graphs, Y, epochs=2)
    oc.fit(twin, graphs, Y)
    oc.fit(twin, graphs, Y, indices=range(G // 2), threads=3)
    oc.fit(twin, graphs, Y, indices=range(G // 2, G), threads=3)
    assert twin.step == model.step
    assert np.array_equal(twin.clause_weights, model.clause_weights)
    assert np.array_equal(twin.ta_state, model.ta_state)
    for a, b in zip(twin.message_ta_state, model.message_ta_state):
        assert np.array_equal(a, b)
