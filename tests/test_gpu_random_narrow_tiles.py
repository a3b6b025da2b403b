"""Randomised differential test of inference on tiles of 33 to 2,000 nodes per graph: data sets, models
(depth 1 to 3, message sizes 32 to 1,024), states (random clauses, clauses of negated literals that hold
wherever their node type is, with up to 300 negated message literals) and the library's switches for the
kernels of such tiles drawn from a seed; the class sums against the C oracle.

Bar: bit-exact (integer work)."""

import numpy as np
import pytest

from oracle import gtm_oracle_c as oc
from tests import helpers

pytestmark = pytest.mark.gpu

CASES_PER_TEST = 25

SWITCHES = [(), (("GTM_MESSAGES_IN_LDS", "1"),), (("GTM_MESSAGES_IN_LDS", "0"),), (("GTM_NARROW_READS", "128"),),
            (("GTM_NO_HALF_ROWS", "1"),), (("GTM_MESSAGES_IN_LDS", "1"), ("GTM_NARROW_READS", "128")),
            (("GTM_NO_FUSED_MESSAGES", "1"),), (("GTM_MESSAGES_IN_LDS", "0"), ("GTM_NO_FUSED_MESSAGES", "1")),
            (("GTM_NARROW_ROWS_AS_STORED", "1"),), (("GTM_NARROW_IN_ORDER", "1"),)]


def pick(rng, xs):
    return xs[int(rng.integers(len(xs)))]


def draw_case(seed):
    rng = np.random.default_rng(seed)
    max_nodes = pick(rng, [33, 64, 100, 200, 361, 500, 700, 841, 1000, 1024, 1500, 2000])
    n_graphs = int(rng.integers(1, 9 if max_nodes > 700 else 20))
    g = dict(n_graphs=n_graphs, max_nodes=max_nodes, min_nodes=int(rng.integers(0 if seed % 4 == 0 else 1, max_nodes + 1)),
             hv_size=pick(rng, [32, 64, 128, 352]), hv_bits=int(rng.integers(1, 3)), n_symbols=int(rng.integers(4, 12)),
             node_types=tuple("t%d" % i for i in range(int(rng.integers(1, 4)))),
             edge_types=tuple("e%d" % i for i in range(int(rng.integers(1, 5)))), max_degree=int(rng.integers(0, 5)))
    depth = pick(rng, [1, 2, 2, 3, 3])
    m = dict(classes=int(rng.integers(2, 8)), clauses=pick(rng, [3, 10, 64, 100, 150, 257]),
             message_size=pick(rng, [32, 64, 96, 128, 256, 512, 1024]), message_bits=int(rng.integers(1, 4)))
    return rng, g, m, depth


@pytest.mark.parametrize("first_seed", range(5000, 5000 + 4 * CASES_PER_TEST, CASES_PER_TEST))
def test_random_narrow_tiles_match_the_oracle(first_seed, tune):
    from tests.gpu_harness import Device

    for seed in range(first_seed, first_seed + CASES_PER_TEST):
        rng, g, m, depth = draw_case(seed)
        graphs = helpers.random_graphs(seed, **g)
        if graphs.max_number_of_graph_nodes == 0:
            continue
        cfg = helpers.oracle_config(graphs, **m, depth=depth)
        hv, M = graphs.hypervector_size, m["message_size"]
        model = helpers.random_model(seed, cfg, depth, include_density=pick(rng, [0.5 / hv, 1.5 / hv, 4.0 / hv]),
                                     message_density=pick(rng, [0.0, 0.002, 0.01]))
        top = cfg.state_bits - 1
        unused = np.setdiff1d(np.arange(hv), np.unique(graphs.hypervectors))
        for c in range(0, cfg.clauses, 3):
            model.ta_state[c, :, top] = 0
            for k in rng.permutation(unused)[: int(rng.integers(0, len(unused) + 1))]:
                lit = hv + int(k)
                model.ta_state[c, lit // 32, top] |= np.uint32(1 << (lit % 32))
            for bank in model.message_ta_state:
                bank[c, :, top] = 0
                for p in rng.permutation(M)[: int(rng.integers(0, min(M, 300)))]:
                    lit = M + int(p)
                    bank[c, lit // 32, top] |= np.uint32(1 << (lit % 32))
        switches = SWITCHES[seed % len(SWITCHES)]
        for name, value in switches:
            tune(name, value)
        what = "seed %d: %r %r depth %d switches %r" % (seed, g, m, depth, switches)
        dev = Device(model, graphs)
        G = graphs.number_of_graphs
        want = oc.score(model, graphs, threads=min(8, oc.threads_available()))
        dev.declare_complementary()
        if dev.build_tiles():
            assert np.array_equal(dev.score(0, G, G), want), "inference on tiles, " + what
            assert np.array_equal(dev.score(0, G, 2), want), "inference on tiles in groups of 2, " + what
        for name, _ in switches:
            tune(name, None)
