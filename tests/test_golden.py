"""The committed fixture tests/golden/frozen_cases.npz (inputs and expected outputs as plain arrays,
written by tests/golden/make_fixtures.py): the NumPy oracle, the C restatement and the HIP path each
reproduce the class sums before training, the state after one pass of training and the class sums
after it.  The data sets are rebuilt from the arrays alone, not from the generator that made them."""

import os
import types

import numpy as np
import pytest

from oracle import gtm_oracle as o
from oracle import gtm_oracle_c as oc

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "frozen_cases.npz")
GRAPH_ARRAYS = ("X", "node_type", "number_of_graph_node_edges", "edge", "node_index", "edge_index",
                "number_of_graph_nodes")


def load_case(i):
    z = np.load(PATH, allow_pickle=False)
    assert i < int(z["n_cases"])
    p = "c%d_" % i
    gs = z[p + "graph_scalars"]
    graphs = types.SimpleNamespace(**{name: z[p + name] for name in GRAPH_ARRAYS})
    graphs.number_of_graphs, graphs.max_number_of_graph_nodes, graphs.number_of_nodes = int(gs[0]), int(gs[1]), int(gs[2])
    n_types = int(gs[3])
    graphs.number_of_node_types = lambda: n_types
    graphs.hypervector_size = int(gs[4])
    graphs.signature = "frozen case %d" % i
    c = [int(v) for v in z[p + "config"]]
    cfg = o.Config(classes=c[0], clauses=c[1], literals=c[2], state_bits=c[3], boost_true_positive_feedback=c[4],
                   threshold=c[5], q=float(z[p + "q"]), max_included_literals=c[6], negative_clauses=c[7],
                   max_nodes=c[8], message_size=c[9], message_bits=c[10])
    depth, seed = c[11], c[12]
    model = o.Model(cfg, depth, tuple(float(v) for v in z[p + "s"]), z[p + "ta_state"].copy(),
                    [z[p + "bank%d" % l].copy() for l in range(depth - 1)], z[p + "clause_weights"].copy(),
                    z[p + "hypervectors"].copy(), seed, 0)
    want = dict(sums_before=z[p + "sums_before"], ta_after=z[p + "ta_after"],
                banks_after=[z[p + "bank%d_after" % l] for l in range(depth - 1)],
                weights_after=z[p + "weights_after"], sums_after=z[p + "sums_after"])
    return graphs, model, z[p + "encoded_Y"], want


def check(model_state, want):
    ta, banks, weights = model_state
    assert np.array_equal(weights, want["weights_after"])
    assert np.array_equal(ta, want["ta_after"])
    assert len(banks) == len(want["banks_after"])
    for got, expected in zip(banks, want["banks_after"]):
        assert np.array_equal(got, expected)


CASES = [0, 1, 2]


def test_the_fixture_is_not_trivial():
    for i in CASES:
        graphs, model, Y, want = load_case(i)
        assert (want["ta_after"] != model.ta_state).sum() > 100
        assert (want["weights_after"] != model.clause_weights).any()
        assert not np.array_equal(want["sums_before"], want["sums_after"])
        assert want["sums_before"].shape == (graphs.number_of_graphs, model.cfg.classes)


@pytest.mark.parametrize("case", CASES)
def test_numpy_oracle_reproduces_the_fixture(case):
    graphs, model, Y, want = load_case(case)
    assert np.array_equal(o.score(model, graphs), want["sums_before"])
    o.fit(model, graphs, Y)
    check((model.ta_state, model.message_ta_state, model.clause_weights), want)
    assert np.array_equal(o.score(model, graphs), want["sums_after"])


@pytest.mark.parametrize("case", CASES)
def test_c_oracle_reproduces_the_fixture(case):
    if not (oc.available() or oc.build()):
        pytest.skip("no C compiler")
    graphs, model, Y, want = load_case(case)
    assert np.array_equal(oc.score(model, graphs), want["sums_before"])
    oc.fit(model, graphs, Y, threads=2)
    check((model.ta_state, model.message_ta_state, model.clause_weights), want)
    assert np.array_equal(oc.score(model, graphs), want["sums_after"])


@pytest.mark.gpu
@pytest.mark.parametrize("tiles", [False, True], ids=["plain", "tiles"])
@pytest.mark.parametrize("case", CASES)
def test_hip_path_reproduces_the_fixture(case, tiles):
    from tests.gpu_harness import Device

    graphs, model, Y, want = load_case(case)
    dev = Device(model, graphs)
    if tiles and not dev.build_tiles():
        pytest.skip("no tile layout for this shape")
    G = graphs.number_of_graphs
    assert np.array_equal(dev.score(0, G, G), want["sums_before"])
    dev.fit(Y, 0, G, 0)
    ta, banks, w = dev.download()
    check((ta, banks, w), want)
    assert np.array_equal(dev.score(0, G, G), want["sums_after"])
    assert np.array_equal(dev.score(0, G, 5), want["sums_after"])
