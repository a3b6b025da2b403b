"""Randomised differential test: the HIP path against the CPU oracle on random small
shapes — data sets (ragged graphs, graphs without nodes, node and edge types, degrees),
models (classes, clauses, depth, message size and bits, state bits, feedback options) and
states (include densities) drawn from a seed.  Per case: inference through the
per-operator kernels and on tiles (one and several launch groups), one epoch of training,
inference on the trained state.

Bar: bit-exact (integer work)."""

import numpy as np
import pytest

from oracle import gtm_oracle as o
from tests import helpers

pytestmark = pytest.mark.gpu

CASES_PER_TEST = 20


def pick(rng, xs):
    return xs[int(rng.integers(len(xs)))]


def draw_case(seed):
    rng = np.random.default_rng(seed)
    max_nodes = pick(rng, [1, 2, 3, 8, 31, 32, 33, 64, 65, 100, 200, 361])
    n_graphs = int(rng.integers(1, 25 if max_nodes <= 65 else 8))
    g = dict(n_graphs=n_graphs, max_nodes=max_nodes, min_nodes=int(rng.integers(0 if seed % 3 == 0 else 1, max_nodes + 1)),
             hv_size=pick(rng, [8, 16, 20, 32, 40, 64, 100, 128, 300]), hv_bits=int(rng.integers(1, 4)),
             n_symbols=int(rng.integers(4, 30)),
             node_types=tuple("t%d" % i for i in range(int(rng.integers(1, 4)))),
             edge_types=tuple("e%d" % i for i in range(int(rng.integers(1, 5)))),
             max_degree=int(rng.integers(0, 5)))
    depth = pick(rng, [1, 1, 2, 2, 3, 4])
    m = dict(classes=int(rng.integers(2, 12)), clauses=pick(rng, [1, 3, 10, 33, 64, 100, 257]),
             message_size=pick(rng, [8, 16, 32, 37, 64, 96, 128, 256]), message_bits=int(rng.integers(1, 4)),
             state_bits=pick(rng, [4, 5, 8, 8, 8, 12]), boost=int(rng.integers(0, 2)),
             max_included=pick(rng, [None, None, 3, 9, 40]), T=int(rng.integers(5, 100)))
    density = pick(rng, [0.0007, 0.005, 0.02, 0.05, 0.15])
    message_density = pick(rng, [0.0, 0.01, 0.05])
    s = tuple(float(x) for x in np.round(rng.uniform(1.0, 8.0, size=depth), 2))
    return rng, g, m, depth, density, message_density, s


@pytest.mark.parametrize("first_seed", range(1000, 1000 + 10 * CASES_PER_TEST, CASES_PER_TEST))
def test_random_shapes_match_the_oracle(first_seed):
    from tests.gpu_harness import Device

    for seed in range(first_seed, first_seed + CASES_PER_TEST):
        rng, g, m, depth, density, message_density, s = draw_case(seed)
        graphs = helpers.random_graphs(seed, **g)
        if graphs.max_number_of_graph_nodes == 0:
            continue  # a data set without a single node has no node types and no model
        what = "seed %d: %r %r depth %d densities %g %g s %r" % (seed, g, m, depth, density, message_density, s)
        cfg = helpers.oracle_config(graphs, **m, depth=depth)
        model = helpers.random_model(seed, cfg, depth, s=s if depth > 1 else s[0], include_density=density,
                                     message_density=message_density)
        dev = Device(model, graphs)
        G = graphs.number_of_graphs
        want = o.score(model, graphs)
        assert np.array_equal(dev.score(0, G, G), want), "per-operator inference, " + what
        if dev.build_tiles():
            assert np.array_equal(dev.score(0, G, G), want), "inference on tiles, " + what
            assert np.array_equal(dev.score(0, G, 3), want), "inference on tiles in groups of 3, " + what
        Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, 0)
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights, " + what
        assert np.array_equal(ta, model.ta_state), "layer-0 automata, " + what
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d, %s" % (layer + 1, what)
        assert np.array_equal(dev.score(0, G, G), o.score(model, graphs)), "inference after training, " + what
