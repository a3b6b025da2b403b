"""HIP path vs the CPU oracle, one operator at a time, through the C ABI.

Bar: bit-exact (everything here is integer / bitwise work)."""

import copy
import ctypes

import numpy as np
import pytest

from graphtsetlinmachine_amd import _abi
from oracle import gtm_oracle as o
from tests import helpers

pytestmark = pytest.mark.gpu

SHAPES = [
    # seed, graphs kwargs, model kwargs
    dict(seed=1, g=dict(n_graphs=5, max_nodes=40, hv_size=20), m=dict(classes=3, clauses=70, depth=1)),
    dict(seed=2, g=dict(n_graphs=4, max_nodes=70, hv_size=16, node_types=("a", "b"), edge_types=("x", "y", "z")),
         m=dict(classes=2, clauses=33, depth=2, message_size=37)),
    dict(seed=3, g=dict(n_graphs=3, max_nodes=32, hv_size=64, min_nodes=32), m=dict(classes=4, clauses=300, depth=3,
                                                                                  message_size=64, message_bits=3)),
    dict(seed=4, g=dict(n_graphs=6, max_nodes=3, hv_size=300, hv_bits=3, n_symbols=9),
         m=dict(classes=5, clauses=20, depth=2, message_size=16, message_bits=1, state_bits=4)),
]


def build(shape, include_density=0.03):
    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(1.0, 3.0, 2.0)[:depth], include_density=include_density)
    return graphs, cfg, model


def graph_slices(graphs, e):
    n = int(graphs.number_of_graph_nodes[e])
    base = int(graphs.node_index[e])
    n_edges = graphs.number_of_graph_node_edges[base:base + n]
    e0 = int(graphs.edge_index[base]) if n else 0
    edge = graphs.edge[e0:e0 + int(n_edges.astype(np.int64).sum())]
    return n, base, n_edges, edge


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "shape%d" % s["seed"])
@pytest.mark.parametrize("density", [0.0, 0.03, 0.5])
def test_inference_operators(shape, density):
    from tests.gpu_harness import Device, host

    graphs, cfg, model = build(shape, density)
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    bitmap, n_incl = dev.calculate_messages(0, G)
    h_bitmap = host(bitmap, np.uint32, (G, cfg.clauses, cfg.node_chunks))
    h_incl = host(n_incl, np.int32, (cfg.clauses,))
    expect = []
    for e in range(G):
        n, base, n_edges, edge = graph_slices(graphs, e)
        bm, incl = o.calculate_messages(cfg, model.ta_state, graphs.node_type[base:base + n],
                                        graphs.number_of_node_types(), n, graphs.X[base:base + n])
        expect.append(bm)
        assert np.array_equal(h_bitmap[e], bm), "calculate_messages graph %d" % e
    assert np.array_equal(h_incl, incl)

    cur, cur_host = bitmap, np.stack(expect)
    for layer in range(model.depth - 1):
        cx = dev.exchange_messages(0, G, cur)
        h_cx = host(cx, np.uint32, (G, cfg.max_nodes, cfg.message_chunks))
        nxt = dev.calculate_messages_conditional(0, G, layer, cur, n_incl, cx)
        h_nxt = host(nxt, np.uint32, (G, cfg.clauses, cfg.node_chunks))
        new_host = []
        for e in range(G):
            n, base, n_edges, edge = graph_slices(graphs, e)
            want_cx = o.build_messages(cfg, n, model.hypervectors, cur_host[e], n_edges, edge)
            assert np.array_equal(h_cx[e, :n], want_cx), "messages layer %d graph %d" % (layer, e)
            bm, incl = o.calculate_messages_conditional(
                cfg, model.message_ta_state[layer], graphs.node_type[base:base + n], graphs.number_of_node_types(),
                n, cur_host[e], np.zeros(cfg.clauses, dtype=np.int32), want_cx)
            assert np.array_equal(h_nxt[e], bm), "conditional layer %d graph %d" % (layer, e)
            new_host.append(bm)
        cur, cur_host = nxt, np.stack(new_host)

    sums = host(dev.evaluate(0, G, cur), np.int32, (G, cfg.classes))
    for e in range(G):
        n = int(graphs.number_of_graph_nodes[e])
        assert np.array_equal(sums[e], o.evaluate(cfg, cur_host[e], model.clause_weights, n))
    # the whole driver loop, at two batch sizes
    want = o.score(model, graphs)
    assert np.array_equal(dev.score(0, G, G), want)
    assert np.array_equal(dev.score(1, G - 1, 2), want[1:])


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "shape%d" % s["seed"])
def test_include_counts_accumulate(shape):
    from tests.gpu_harness import Device, host

    graphs, cfg, model = build(shape, 0.1)
    if model.depth < 2:
        pytest.skip("needs a message layer")
    dev = Device(model, graphs)
    bitmap, n_incl = dev.calculate_messages(0, 1)
    cx = dev.exchange_messages(0, 1, bitmap)
    dev.calculate_messages_conditional(0, 1, 0, bitmap, n_incl, cx)
    inc0 = o._popcount32(o._include_plane(model.ta_state, cfg.state_bits, cfg.filter)).sum(axis=1)
    inc1 = o._popcount32(o._include_plane(model.message_ta_state[0], cfg.state_bits, cfg.message_filter)).sum(axis=1)
    assert np.array_equal(host(n_incl, np.int32, (cfg.clauses,)), inc0 + inc1)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "shape%d" % s["seed"])
@pytest.mark.parametrize("boost,max_included", [(1, None), (0, None), (1, 3)])
def test_training_operators(shape, boost, max_included):
    from tests.gpu_harness import Device, host
    from graphtsetlinmachine_amd.tm import _to_device

    graphs, cfg, model = build(shape, 0.03)
    cfg.boost_true_positive_feedback = boost
    if max_included is not None:
        cfg.max_included_literals = max_included
    dev = Device(model, graphs)
    rng = np.random.default_rng(shape["seed"])
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=graphs.number_of_graphs), cfg.classes, cfg.threshold)
    for e in range(graphs.number_of_graphs):
        step = 1000 + e
        n, base, n_edges, edge = graph_slices(graphs, e)
        ref = copy.deepcopy(model)
        bitmap, class_sum, n_incl, layers = o.evaluate_graph(ref, graphs, e)
        d_bitmap = _to_device(bitmap)

        want_node = o.select_clause_node(cfg, model.seed, step, bitmap, n)
        got_node = dev.select_clause_node(e, step, d_bitmap)
        assert np.array_equal(host(got_node, np.int32, (cfg.clauses,)), want_node)

        weights = model.clause_weights.copy()
        want_upd = o.select_clause_updates(cfg, model.seed, step, weights, class_sum, Y[e], want_node)
        got_upd = dev.select_clause_updates(step, _to_device(class_sum), Y, e, got_node)
        assert np.array_equal(host(got_upd, np.int32, (cfg.classes, cfg.clauses)), want_upd)
        assert np.array_equal(host(dev.weights, np.int32, weights.shape), weights)

        d_incl = _to_device(n_incl)
        ta = model.ta_state.copy()
        o.update(cfg, model.seed, step, model.s[0], ta, want_node, n_incl, graphs.X[base:base + n], want_upd)
        dev.update(e, step, got_node, d_incl, got_upd)
        got_ta, got_banks, _ = dev.download()
        assert np.array_equal(got_ta, ta), "update graph %d" % e
        for layer in range(model.depth - 1):
            bank = model.message_ta_state[layer].copy()
            o.update_message(cfg, model.seed, step, layer + 1, model.s[layer + 1], bank, want_node, n_incl,
                             layers[layer], want_upd)
            cx = np.zeros((cfg.max_nodes, cfg.message_chunks), dtype=np.uint32)
            cx[:n] = layers[layer]
            dev.update_message(step, layer + 1, got_node, d_incl, _to_device(cx), got_upd)
            assert np.array_equal(dev.download()[1][layer], bank), "update_message graph %d layer %d" % (e, layer)
            model.message_ta_state[layer] = bank
        model.ta_state = ta
        model.clause_weights = weights


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "shape%d" % s["seed"])
@pytest.mark.parametrize("tiles", [False, True], ids=["plain", "tiles"])
def test_fit_trajectory_bit_exact(shape, tiles):
    """gtm_fit over a few epochs leaves exactly the oracle's automata and weights
    (with tiles, the fused training steps run instead of one launch per operator)."""
    from tests.gpu_harness import Device

    graphs, cfg, model = build(shape, 0.02)
    dev = Device(model, graphs)
    if tiles:
        assert dev.build_tiles()
    rng = np.random.default_rng(shape["seed"] + 100)
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=graphs.number_of_graphs), cfg.classes, cfg.threshold)
    G = graphs.number_of_graphs
    for epoch in range(3):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(model.depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


def test_prepare_matches_oracle():
    import ctypes
    from tests.gpu_harness import abi_config, dev_u32, host
    from graphtsetlinmachine_amd import _abi
    from graphtsetlinmachine_amd.tm import _ptr, _stream

    cfg = o.Config(classes=3, clauses=77, literals=40, state_bits=6, max_nodes=5, message_size=19)
    acfg = abi_config(cfg, 2, 1.0, seed=0xDEADBEEFCAFE)
    ta = dev_u32((cfg.clauses, cfg.la_chunks, cfg.state_bits))
    w = dev_u32((cfg.classes, cfg.clauses))
    bank = dev_u32((cfg.clauses, cfg.message_chunks, cfg.state_bits))
    _abi.call("gtm_prepare", ctypes.byref(acfg), 5, _ptr(ta), _ptr(w), _stream())
    _abi.call("gtm_prepare_message_ta_state", ctypes.byref(acfg), _ptr(bank), _stream())
    want_ta, want_w = o.prepare(cfg, 0xDEADBEEFCAFE, 5)
    assert np.array_equal(host(ta, np.uint32, want_ta.shape), want_ta)
    assert np.array_equal(host(w, np.int32, want_w.shape), want_w)
    assert np.array_equal(host(bank, np.uint32, (cfg.clauses, cfg.message_chunks, cfg.state_bits)),
                          o.prepare_message_ta_state(cfg))
    assert set(np.unique(want_w)) == {-1, 1}


def test_bad_arguments_are_reported():
    import ctypes
    from tests.gpu_harness import abi_config
    from graphtsetlinmachine_amd import _abi

    cfg = o.Config(classes=2, clauses=4, literals=8, max_nodes=2)
    acfg = abi_config(cfg, 1, 1.0, 1)
    with pytest.raises(_abi.GtmError, match="NULL"):
        _abi.call("gtm_prepare", ctypes.byref(acfg), 0, None, None, None)
    acfg.state_bits = 40
    with pytest.raises(_abi.GtmError, match="state_bits"):
        _abi.call("gtm_prepare_message_ta_state", ctypes.byref(acfg), None, None)


TILE_SHAPES = [
    # tiny graphs (several per word), one word, several words, exactly 64 words, more than one node type
    dict(seed=11, g=dict(n_graphs=300, max_nodes=1, hv_size=40), classes=3, clauses=50),
    dict(seed=12, g=dict(n_graphs=200, max_nodes=3, hv_size=16, node_types=("a", "b")), classes=2, clauses=64),
    # many literals: the tile narrows until its rows fit in LDS
    dict(seed=20, g=dict(n_graphs=150, max_nodes=1, hv_size=1500, n_symbols=40), classes=3, clauses=40),
    dict(seed=21, g=dict(n_graphs=90, max_nodes=2, hv_size=700, n_symbols=30), classes=10, clauses=50),
    dict(seed=13, g=dict(n_graphs=70, max_nodes=16, min_nodes=9, hv_size=20), classes=4, clauses=33),
    dict(seed=14, g=dict(n_graphs=40, max_nodes=31, min_nodes=17, hv_size=64), classes=10, clauses=200),
    dict(seed=15, g=dict(n_graphs=23, max_nodes=361, min_nodes=300, hv_size=128, max_degree=0), classes=10, clauses=120),
    dict(seed=16, g=dict(n_graphs=5, max_nodes=2048, min_nodes=1990, hv_size=16, max_degree=0, node_types=("a", "b", "c")),
         classes=2, clauses=40),
    # 5 literal words per node (layer 0 in two phases, nodes tested word-parallel)
    dict(seed=19, g=dict(n_graphs=25, max_nodes=90, min_nodes=30, hv_size=80, n_symbols=12, node_types=("a", "b")),
         classes=3, clauses=70),
    # 12 and 16 literal words per node (layer 0 in two phases)
    dict(seed=17, g=dict(n_graphs=30, max_nodes=100, min_nodes=20, hv_size=192, n_symbols=12), classes=3, clauses=90),
    dict(seed=18, g=dict(n_graphs=20, max_nodes=50, hv_size=256, n_symbols=12, node_types=("a", "b")), classes=4,
         clauses=64),
]


@pytest.mark.parametrize("shape", TILE_SHAPES, ids=lambda s: "tiles%d" % s["seed"])
@pytest.mark.parametrize("density", [0.0, 0.02, 0.2])
def test_tile_scoring_equals_oracle(shape, density):
    """Depth-1 gtm_score on literal-major tiles == oracle == the bitmap path."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"])
    model = helpers.random_model(shape["seed"], cfg, 1, include_density=density)
    model.ta_state[3, :, cfg.state_bits - 1] = 0  # an empty clause among the random ones
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    plain = dev.score(0, G, G)
    assert dev.build_tiles(), "this shape should have a tile layout"
    tiled = dev.score(0, G, G)
    assert np.array_equal(tiled, plain)
    sample = sorted(set([0, 1, G // 2, G - 1]))
    want = o.score(model, graphs, sample)
    assert np.array_equal(tiled[sample], want)
    # a range that starts and ends inside tiles
    if G > 7:
        assert np.array_equal(dev.score(3, G - 5, G), plain[3:G - 2])


@pytest.mark.parametrize("hv_size,sizes", [
    (64, [40, 0, 2, 64, 1, 50, 3, 1, 2, 5]), (128, [361, 1, 300, 0, 2, 361, 3, 1]), (256, [100, 1, 31, 2, 90, 1, 3, 2, 1]),
    (80, [70, 1, 0, 2, 33, 64, 1, 3]), (1100, [40, 1, 2, 35, 0, 1])])  # 5 and 69 literal words per node: the other two-phase kernel
@pytest.mark.parametrize("depth", [1, 2])
def test_tile_scoring_with_clauses_of_negated_literals(hv_size, sizes, depth):
    """Clauses that include 16 to 40 negated literals and nothing else: each
    of them holds at nearly every node, so the rarest literals of a clause
    filter out almost nothing and the two-phase layer 0 is left with most node
    slots (it then ANDs the rows of all the clause's literals instead)."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(41, n_graphs=len(sizes), hv_size=hv_size, n_symbols=24, sizes=sizes, max_degree=2)
    cfg = helpers.oracle_config(graphs, classes=3, clauses=48, depth=depth, message_size=64)
    model = helpers.random_model(41, cfg, depth, include_density=0.0, message_density=0.0)
    rng = np.random.default_rng(41)
    top = cfg.state_bits - 1
    used = np.unique(graphs.hypervectors)  # the bits that symbols set: their negations are what tells nodes apart
    for c in range(cfg.clauses):
        n = int(rng.integers(16, 41))
        bits = rng.permutation(used)[:n]
        if len(bits) < n:
            bits = np.concatenate([bits, rng.choice(np.setdiff1d(np.arange(hv_size), used), size=n - len(bits), replace=False)])
        for k in bits:
            lit = hv_size + int(k)
            model.ta_state[c, lit // 32, top] |= np.uint32(1 << (lit % 32))
    G = graphs.number_of_graphs
    want = o.score(model, graphs)
    assert len(np.unique(want, axis=0)) > 1, "the clauses should tell some graphs apart"
    dev = Device(model, graphs)
    assert np.array_equal(dev.score(0, G, G), want)
    assert dev.build_tiles()
    assert np.array_equal(dev.score(0, G, G), want)
    assert np.array_equal(dev.score(0, G, 2), want)


DEEP_TILE_SHAPES = [
    # several graphs per word; one word per graph; several words; 361-node graphs; literal rows too
    # big for LDS (read in place); graphs without nodes; single-node graphs with self-loops
    dict(seed=31, g=dict(n_graphs=120, max_nodes=3, hv_size=16, node_types=("a", "b"), edge_types=("x", "y", "z")),
         m=dict(classes=2, clauses=33, depth=2, message_size=37)),
    dict(seed=32, g=dict(n_graphs=60, max_nodes=16, min_nodes=9, hv_size=20),
         m=dict(classes=4, clauses=100, depth=3, message_size=64, message_bits=3)),
    dict(seed=33, g=dict(n_graphs=30, max_nodes=70, hv_size=16, edge_types=("x", "y")),
         m=dict(classes=3, clauses=70, depth=2, message_size=37)),
    dict(seed=34, g=dict(n_graphs=12, max_nodes=361, min_nodes=300, hv_size=128, edge_types=("l", "r", "u", "d")),
         m=dict(classes=10, clauses=80, depth=2, message_size=256)),
    dict(seed=35, g=dict(n_graphs=5, sizes=[3, 520, 40, 1, 200], hv_size=1500, n_symbols=30),
         m=dict(classes=2, clauses=60, depth=2, message_size=32), density=0.0007),
    dict(seed=36, g=dict(n_graphs=7, hv_size=16, sizes=[5, 0, 33, 1, 0, 40, 0]),
         m=dict(classes=3, clauses=20, depth=3, message_size=16, message_bits=1)),
    dict(seed=37, g=dict(n_graphs=200, max_nodes=1, hv_size=40), m=dict(classes=3, clauses=50, depth=2, message_size=8)),
]


@pytest.mark.parametrize("shape", DEEP_TILE_SHAPES, ids=lambda s: "tiles%d" % s["seed"])
@pytest.mark.parametrize("message_density", [0.0, 0.01, 0.1, 0.6])
@pytest.mark.parametrize("messages", ["graph-per-workgroup", "graph-per-workgroup-lists-by-scalar-loads",
                                      "three-launches", "three-launches-atomics"])
def test_tile_scoring_with_message_layers(shape, message_density, messages, tune):
    """gtm_score with message layers on literal-major tiles == oracle == the bitmap path, with the
    message rows built by one workgroup per graph (where the shape allows) and by the three
    launches that keep the vectors in global memory.  The clause lists of the message layers reach the
    evaluating waves through LDS (lists of up to 256 entries: at density 0.6 the larger message sizes
    have longer ones, which take scalar loads) or, switched off, all by scalar loads."""
    from tests.gpu_harness import Device

    if not messages.startswith("graph-per-workgroup"):
        tune("GTM_NO_FUSED_MESSAGES", "1")
    if messages == "graph-per-workgroup-lists-by-scalar-loads":
        tune("GTM_NO_LISTS_IN_LDS", "1")
    if messages == "three-launches-atomics":
        tune("GTM_NODE_MESSAGES_BY_ATOMICS", "1")

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth)
    model = helpers.random_model(shape["seed"], cfg, depth, include_density=shape.get("density", 0.02),
                                 message_density=message_density)
    model.ta_state[3, :, cfg.state_bits - 1] = 0  # an empty clause among the random ones
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    plain = dev.score(0, G, G)
    assert dev.build_tiles(), "this shape should have a tile layout"
    tiled = dev.score(0, G, G)
    assert np.array_equal(tiled, plain)
    sample = sorted(set(e for e in (0, 1, 2, 3, 4, G // 2, G - 1) if e < G))
    assert np.array_equal(tiled[sample], o.score(model, graphs, sample))
    # several launch groups; a range that starts and ends inside tiles
    assert np.array_equal(dev.score(0, G, 3), plain)
    if G > 7:
        assert np.array_equal(dev.score(3, G - 5, 5), plain[3:G - 2])


@pytest.mark.parametrize("shape", DEEP_TILE_SHAPES, ids=lambda s: "tiles%d" % s["seed"])
@pytest.mark.parametrize("boost,max_included,state_bits", [(1, None, 8), (0, 9, 5)])
@pytest.mark.parametrize("messages", ["by-node-vectors", "by-scatter"])
def test_fused_fit_with_message_layers(shape, boost, max_included, state_bits, messages, tune):
    """The fused training step of models with message layers == the oracle: automata of every
    bank and the weights after each of two epochs.  Both ways of building the messages (per-node
    bit vectors rotated along the edges, taken when MESSAGE_SIZE is a multiple of 32; one scatter
    per true clause, node and edge) are forced in turn."""
    from tests.gpu_harness import Device

    tune("GTM_FIT_FACTOR_MIN", "0" if messages == "by-node-vectors" else str(1 << 60))
    tune("GTM_NO_SMALL_FIT", "1")  # the one-workgroup kernel has its own test
    tune("GTM_NO_DEEP_PERSISTENT_FIT", "1")  # and so has the one-launch kernel

    g = dict(shape["g"])
    if "sizes" not in g:
        g["n_graphs"] = min(g["n_graphs"], 12)
    graphs = helpers.random_graphs(shape["seed"], **g)
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth, T=30, boost=boost, max_included=max_included,
                                state_bits=state_bits)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0, 2.0, 1.5)[:depth],
                                 include_density=shape.get("density", 0.02), message_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    rng = np.random.default_rng(shape["seed"])
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    for epoch in range(2):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


ONE_LAUNCH_DEEP_SHAPES = [
    # (every MESSAGE_SIZE a multiple of 32) several graphs per word with node and edge types; three layers;
    # two truth words per graph; 361-node graphs with four edge types, more clauses than one workgroup
    # per clause can hold; graphs without nodes among others, four layers; single nodes with self-loops;
    # no edges at all; several messages bits per clause and a large hypervector
    dict(seed=61, g=dict(n_graphs=40, max_nodes=3, hv_size=16, node_types=("a", "b"), edge_types=("x", "y", "z")),
         m=dict(classes=2, clauses=33, depth=2, message_size=64)),
    dict(seed=62, g=dict(n_graphs=24, max_nodes=16, min_nodes=9, hv_size=20),
         m=dict(classes=4, clauses=100, depth=3, message_size=64, message_bits=3)),
    dict(seed=63, g=dict(n_graphs=10, max_nodes=64, min_nodes=40, hv_size=40, edge_types=("l", "r", "u", "d"),
                         node_types=("a", "b")),
         m=dict(classes=3, clauses=70, depth=2, message_size=96)),
    dict(seed=64, g=dict(n_graphs=6, max_nodes=361, min_nodes=300, hv_size=128, edge_types=("l", "r", "u", "d")),
         m=dict(classes=10, clauses=700, depth=2, message_size=256)),
    dict(seed=65, g=dict(n_graphs=8, hv_size=16, sizes=[5, 0, 33, 1, 0, 40, 64, 0]),
         m=dict(classes=3, clauses=20, depth=4, message_size=32, message_bits=1)),
    dict(seed=66, g=dict(n_graphs=30, max_nodes=1, hv_size=40), m=dict(classes=3, clauses=50, depth=2, message_size=32)),
    dict(seed=67, g=dict(n_graphs=12, max_nodes=40, min_nodes=20, hv_size=100, max_degree=0),
         m=dict(classes=5, clauses=64, depth=2, message_size=128)),
    dict(seed=68, g=dict(n_graphs=16, max_nodes=30, min_nodes=2, hv_size=24, edge_types=("p", "q")),
         m=dict(classes=2, clauses=300, depth=3, message_size=512, message_bits=4)),
]


@pytest.mark.parametrize("shape", ONE_LAUNCH_DEEP_SHAPES, ids=lambda s: "deep%d" % s["seed"])
@pytest.mark.parametrize("boost,max_included,state_bits", [(1, None, 8), (0, 9, 5), (1, None, 12)])
@pytest.mark.parametrize("layout", ["in-lds", "in-lds-40-clauses-per-workgroup", "in-memory", "in-memory-32-row-windows",
                                    "in-memory-40-clauses-per-workgroup", "in-memory-dealt-anew-every-3-examples",
                                    "in-lds-dealt-anew-every-5-examples", "in-memory-clauses-in-order",
                                    "in-memory-70-clauses-per-workgroup"])
def test_one_launch_fit_with_message_layers(shape, boost, max_included, state_bits, layout, tune):
    """A run of training examples of a model with message layers in one cooperative launch
    (k_fit_deep_persistent: clauses spread over workgroups, the nodes' messages and the class sums
    exchanged through device memory): automata of every bank and the weights after each of two
    epochs == the oracle; each epoch is split into two calls, so the state's round trip
    through memory and the restart of the exchange buffers are covered.  Both layouts: automata
    and all rows in LDS; automata in memory with the received rows passing through LDS in windows
    (as wide as fits, and 32 rows wide, so that every layer takes several).  With 40 clauses per
    workgroup what the clauses send is worked out 32 clauses at a time, in two passes.  With several clauses per
    workgroup the clauses are dealt out to the workgroups by their number of literals before every launch; a run is
    then cut into several launches (here: of 3 or 5 examples), or the clauses stay in order."""
    import ctypes
    from tests.gpu_harness import Device
    from graphtsetlinmachine_amd import _abi

    tune("GTM_NO_SMALL_FIT", "1")
    if layout.startswith("in-memory"):
        tune("GTM_FIT_DEEP_IN_MEMORY", "1")
    if layout == "in-memory-32-row-windows":
        tune("GTM_FIT_DEEP_WINDOW_ROWS", "32")
    if layout.endswith("40-clauses-per-workgroup"):
        tune("GTM_FIT_DEEP_CLAUSES_PER_GROUP", "40")
    if layout.endswith("70-clauses-per-workgroup"):
        tune("GTM_FIT_DEEP_CLAUSES_PER_GROUP", "70")
    if "dealt-anew" in layout:
        tune("GTM_FIT_DEEP_CLAUSES_PER_GROUP", "7")
        tune("GTM_FIT_DEEP_CHUNK", "3" if "every-3" in layout else "5")
    if layout.endswith("clauses-in-order"):
        tune("GTM_FIT_DEEP_CLAUSES_PER_GROUP", "7")
        tune("GTM_FIT_DEEP_NO_DEAL", "1")
    kernel = b"k_fit_deep_persistent<in memory>" if layout.startswith("in-memory") else b"k_fit_deep_persistent"
    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth, T=30, boost=boost, max_included=max_included,
                                state_bits=state_bits)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0, 2.0, 1.5, 1.2)[:depth],
                                 include_density=shape.get("density", 0.02), message_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    rng = np.random.default_rng(shape["seed"])
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
    for epoch in range(2):
        o.fit(model, graphs, Y)
        _abi.call("gtm_profile_enable", 1)
        dev.fit(Y, 0, G // 3, epoch * G)
        dev.fit(Y, G // 3, G - G // 3, epoch * G + G // 3)
        _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
        _abi.call("gtm_profile_enable", 0)
        chunk = 3 if "every-3" in layout else 5 if "every-5" in layout else G
        expected = -(-(G // 3) // chunk) + -(-(G - G // 3) // chunk)  # launches of the two calls
        assert (name.value, launches.value) == (kernel, expected), "the one-launch kernel should have run"
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


@pytest.mark.parametrize("layout", ["in-lds", "in-memory"])
def test_one_launch_fit_with_message_layers_gives_up_instead_of_hanging(layout, tune):
    """As for the depth-1 kernel: GTM_FIT_SPIN_LIMIT=abort makes every workgroup give up at its first
    device-wide wait; the kernel drains, the call reports it, every bank and the weights are as
    they were, and the same model trains normally afterwards."""
    from tests.gpu_harness import Device
    from graphtsetlinmachine_amd import _abi

    tune("GTM_NO_SMALL_FIT", "1")
    if layout == "in-memory":
        tune("GTM_FIT_DEEP_IN_MEMORY", "1")
    shape = ONE_LAUNCH_DEEP_SHAPES[1]
    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth, T=30)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0, 2.0, 1.5)[:depth], include_density=0.02,
                                 message_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    G = graphs.number_of_graphs
    Y = o.encode_labels(np.arange(G) % cfg.classes, cfg.classes, cfg.threshold)

    def same_as_oracle():
        ta, banks, w = dev.download()
        return (np.array_equal(w, model.clause_weights) and np.array_equal(ta, model.ta_state) and
                all(np.array_equal(banks[l], model.message_ta_state[l]) for l in range(depth - 1)))

    tune("GTM_FIT_SPIN_LIMIT", "abort")
    with pytest.raises(_abi.GtmError, match="gave up waiting.*as it was before the call"):
        dev.fit(Y, 0, G, 0)
    tune("GTM_FIT_SPIN_LIMIT", None)
    assert same_as_oracle()
    o.fit(model, graphs, Y)
    dev.fit(Y, 0, G, 0)
    assert same_as_oracle()


SMALL_DEEP_SHAPES = [
    # two-node graphs with two edge types; 9..16 nodes, three layers; exactly 64 nodes (two truth
    # words) and four edge types; graphs without nodes among small ones and at the end; single nodes with self-loops;
    # several classes on graphs without edges
    dict(seed=41, g=dict(n_graphs=40, max_nodes=2, min_nodes=2, hv_size=8, edge_types=("x", "y")),
         m=dict(classes=2, clauses=10, depth=2, message_size=256, message_bits=2)),
    dict(seed=42, g=dict(n_graphs=24, max_nodes=16, min_nodes=9, hv_size=20),
         m=dict(classes=4, clauses=100, depth=3, message_size=64, message_bits=3)),
    dict(seed=43, g=dict(n_graphs=10, max_nodes=64, min_nodes=64, hv_size=40, edge_types=("l", "r", "u", "d"),
                         node_types=("a", "b")),
         m=dict(classes=3, clauses=70, depth=2, message_size=96)),
    dict(seed=44, g=dict(n_graphs=8, hv_size=16, sizes=[5, 0, 33, 1, 0, 40, 64, 0]),
         m=dict(classes=3, clauses=20, depth=4, message_size=32, message_bits=1)),
    dict(seed=45, g=dict(n_graphs=30, max_nodes=1, hv_size=40), m=dict(classes=3, clauses=50, depth=2, message_size=32)),
    dict(seed=46, g=dict(n_graphs=12, max_nodes=40, min_nodes=20, hv_size=100, max_degree=0),
         m=dict(classes=5, clauses=64, depth=2, message_size=128)),
]


@pytest.mark.parametrize("shape", SMALL_DEEP_SHAPES, ids=lambda s: "small%d" % s["seed"])
@pytest.mark.parametrize("boost,max_included,state_bits", [(1, None, 8), (0, 9, 5), (1, None, 12)])
def test_one_workgroup_fit_with_message_layers(shape, boost, max_included, state_bits):
    """Small models with message layers on graphs of at most 64 nodes train inside one workgroup
    (k_fit_small): automata of every bank and the weights after each of two epochs == the oracle,
    and the run is split into two calls so the state's round trip through memory is covered."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    m = dict(shape["m"])
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth, T=30, boost=boost, max_included=max_included,
                                state_bits=state_bits)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0, 2.0, 1.5, 1.2)[:depth],
                                 include_density=shape.get("density", 0.02), message_density=0.02)
    dev = Device(model, graphs)
    dev.build_tiles()
    rng = np.random.default_rng(shape["seed"])
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
    for epoch in range(2):
        o.fit(model, graphs, Y)
        _abi.call("gtm_profile_enable", 1)
        dev.fit(Y, 0, G // 2, epoch * G)
        dev.fit(Y, G // 2, G - G // 2, epoch * G + G // 2)
        _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
        _abi.call("gtm_profile_enable", 0)
        assert (name.value, launches.value) == (b"k_fit_small", 2), "the one-workgroup kernel should have run"
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


@pytest.mark.parametrize("shape", TILE_SHAPES, ids=lambda s: "tiles%d" % s["seed"])
@pytest.mark.parametrize("boost,max_included,state_bits", [(1, None, 8), (0, 6, 5)])
@pytest.mark.parametrize("persistent", [True, False], ids=["one-launch", "two-per-graph"])
def test_fused_fit_on_every_tile_geometry(shape, boost, max_included, state_bits, persistent, tune):
    """Both fused depth-1 training paths (one cooperative launch per run of
    examples; two launches per example) == the oracle."""
    from tests.gpu_harness import Device

    if not persistent:
        tune("GTM_NO_PERSISTENT_FIT", "1")

    g = dict(shape["g"])
    g["n_graphs"] = min(g["n_graphs"], 24)
    graphs = helpers.random_graphs(shape["seed"], **g)
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"], T=30, boost=boost,
                                max_included=max_included, state_bits=state_bits)
    model = helpers.random_model(shape["seed"], cfg, 1, s=3.0, include_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    rng = np.random.default_rng(shape["seed"])
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    for epoch in range(2):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, _, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "automata after epoch %d" % epoch
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


MANY_CLASSES_SHAPES = [
    dict(seed=61, g=dict(n_graphs=40, max_nodes=1, hv_size=40, max_degree=0), depth=1, clauses=50),
    dict(seed=62, g=dict(n_graphs=24, max_nodes=31, min_nodes=17, hv_size=64, max_degree=0), depth=1, clauses=90),
    dict(seed=63, g=dict(n_graphs=8, max_nodes=361, min_nodes=300, hv_size=128, max_degree=0), depth=1, clauses=40),
    dict(seed=64, g=dict(n_graphs=30, max_nodes=12, min_nodes=2, hv_size=16, max_degree=2), depth=2, clauses=30),
    dict(seed=65, g=dict(n_graphs=10, max_nodes=150, min_nodes=70, hv_size=32, max_degree=2), depth=3, clauses=40),
]


@pytest.mark.parametrize("shape", MANY_CLASSES_SHAPES, ids=lambda s: "shape%d" % s["seed"])
@pytest.mark.parametrize("state_bits", [1, 2, 16, 17, 32])
def test_narrow_and_wide_automata(shape, state_bits):
    """Automata of 1 to 32 bits (the training kernels keep 8, 16 or 32 planes of a word in
    registers): two epochs on whichever path the shape takes == the oracle."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    depth = shape["depth"]
    cfg = helpers.oracle_config(graphs, classes=4, clauses=shape["clauses"], depth=depth, T=20, message_size=64,
                                state_bits=state_bits)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0,) * depth, include_density=0.03)
    dev = Device(model, graphs)
    dev.build_tiles()
    G = graphs.number_of_graphs
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))
    rng = np.random.default_rng(shape["seed"])
    Y = o.encode_labels(rng.integers(0, 4, size=G), 4, cfg.threshold)
    for epoch in range(2):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


@pytest.mark.parametrize("shape", MANY_CLASSES_SHAPES, ids=lambda s: "shape%d" % s["seed"])
@pytest.mark.parametrize("classes", [65, 130])
def test_more_classes_than_lanes(shape, classes):
    """More classes than a wave has lanes (the kernels keep per-class values lane by lane up to 64
    and loop beyond): inference without and with tiles, two epochs of training on whichever path
    the shape takes, inference again == the oracle."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    depth = shape["depth"]
    cfg = helpers.oracle_config(graphs, classes=classes, clauses=shape["clauses"], depth=depth, T=20, message_size=64)
    model = helpers.random_model(shape["seed"], cfg, depth, s=(3.0,) * depth, include_density=0.03)
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    want = o.score(model, graphs)
    assert np.array_equal(dev.score(0, G, G), want)
    if dev.build_tiles():
        assert np.array_equal(dev.score(0, G, G), want)
        assert np.array_equal(dev.score(0, G, 7), want)
    rng = np.random.default_rng(shape["seed"])
    Y = o.encode_labels(rng.integers(0, classes, size=G), classes, cfg.threshold)
    for epoch in range(2):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


@pytest.mark.parametrize("shape", [TILE_SHAPES[3], TILE_SHAPES[5], TILE_SHAPES[6]], ids=lambda s: "tiles%d" % s["seed"])
@pytest.mark.parametrize("per_group", [1, 3, 16, 20, 40])
def test_one_launch_fit_with_any_number_of_clauses_per_workgroup(shape, per_group, tune):
    """The cooperative training kernel gives a workgroup 8 or more clauses; GTM_FIT_PER_GROUP sets
    the number.  Up to 16 (one clause per wave) a small clause's feedback runs inside its wave,
    above that a wave evaluates several clauses and the feedback is shared out over the group:
    every split == the oracle."""
    from tests.gpu_harness import Device

    tune("GTM_FIT_PER_GROUP", str(per_group))
    g = dict(shape["g"])
    g["n_graphs"] = min(g["n_graphs"], 24)
    graphs = helpers.random_graphs(shape["seed"], **g)
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"], T=30)
    model = helpers.random_model(shape["seed"], cfg, 1, s=3.0, include_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    rng = np.random.default_rng(shape["seed"] + per_group)
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    for epoch in range(2):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, _, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "automata after epoch %d" % epoch
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


@pytest.mark.parametrize("seed,g,m", [
    (15, dict(n_graphs=10, max_nodes=361, min_nodes=300, hv_size=128, max_degree=0), dict(classes=10, clauses=60, depth=1)),
    (18, dict(n_graphs=12, max_nodes=50, hv_size=256, n_symbols=12, node_types=("a", "b")), dict(classes=4, clauses=64, depth=1)),
    (13, dict(n_graphs=20, max_nodes=16, min_nodes=9, hv_size=80), dict(classes=4, clauses=33, depth=1)),
    (34, dict(n_graphs=8, max_nodes=200, min_nodes=100, hv_size=128, edge_types=("l", "r")),
     dict(classes=3, clauses=40, depth=2, message_size=64)),
    (38, dict(n_graphs=6, hv_size=2200, n_symbols=30, sizes=[3, 70, 0, 1, 33, 64]), dict(classes=2, clauses=30, depth=1)),
], ids=lambda v: str(v) if isinstance(v, int) else "")
@pytest.mark.parametrize("density", [0.3, 0.9])
@pytest.mark.parametrize("persistent", [True, False], ids=["one-launch", "per-example"])
def test_fused_fit_with_many_literals(seed, g, m, density, persistent, tune):
    """Clauses with many included literals (the training kernels AND a few of their rows and
    test the surviving nodes against the whole include mask) == the oracle."""
    from tests.gpu_harness import Device

    if not persistent:
        tune("GTM_NO_PERSISTENT_FIT", "1")
    elif m["depth"] > 1:
        pytest.skip("models with message layers have one training path")
    graphs = helpers.random_graphs(seed, **g)
    m = dict(m)
    depth = m.pop("depth")
    cfg = helpers.oracle_config(graphs, **m, depth=depth, T=30)
    model = helpers.random_model(seed, cfg, depth, s=(4.0, 2.0)[:depth], include_density=density, message_density=0.05)
    # dense random includes are almost never satisfied: give a third of the clauses includes that one node satisfies
    rng = np.random.default_rng(seed)
    for c in range(0, cfg.clauses, 3):
        node = int(rng.integers(graphs.number_of_nodes))
        keep = graphs.X[node].copy()
        keep[-1] &= np.uint32(cfg.filter)
        model.ta_state[c, :, cfg.state_bits - 1] &= keep
    dev = Device(model, graphs)
    assert dev.build_tiles()
    G = graphs.number_of_graphs
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    for epoch in range(2):
        o.fit(model, graphs, Y)
        dev.fit(Y, 0, G, epoch * G)
        ta, banks, w = dev.download()
        assert np.array_equal(w, model.clause_weights), "weights after epoch %d" % epoch
        assert np.array_equal(ta, model.ta_state), "layer-0 automata after epoch %d" % epoch
        for layer in range(depth - 1):
            assert np.array_equal(banks[layer], model.message_ta_state[layer]), "bank %d epoch %d" % (layer, epoch)
    assert np.array_equal(dev.score(0, G, G), o.score(model, graphs))


def test_fused_fit_with_an_empty_graph():
    from tests.gpu_harness import Device

    g = helpers.random_graphs(19, n_graphs=6, hv_size=16, sizes=[5, 0, 33, 1, 0, 40])
    cfg = helpers.oracle_config(g, classes=3, clauses=20, T=20)
    model = helpers.random_model(5, cfg, 1, s=2.0, include_density=0.05)
    dev = Device(model, g)
    assert dev.build_tiles()
    Y = o.encode_labels(np.array([0, 1, 2, 0, 1, 2]), 3, cfg.threshold)
    o.fit(model, g, Y, epochs=2)
    dev.fit(Y, 0, 6, 0)
    dev.fit(Y, 0, 6, 6)
    ta, _, w = dev.download()
    assert np.array_equal(w, model.clause_weights) and np.array_equal(ta, model.ta_state)


@pytest.mark.parametrize("hv_size,density", [(16, 0.05), (64, 0.05), (64, 0.3)])
def test_empty_graphs_score_like_the_reference_arithmetic(hv_size, density):
    """A graph without nodes: the reference's chunk arithmetic (C division,
    kernels.py:289-295) leaves every clause true, so it scores sum_c W[k][c]."""
    from tests.gpu_harness import Device

    g = helpers.random_graphs(17, n_graphs=6, hv_size=hv_size, sizes=[5, 0, 33, 1, 0, 40])
    cfg = helpers.oracle_config(g, classes=3, clauses=20)
    model = helpers.random_model(5, cfg, 1, include_density=density)
    want = o.score(model, g)
    assert np.array_equal(want[1], model.clause_weights.sum(axis=1)) and np.array_equal(want[4], want[1])
    dev = Device(model, g)
    assert np.array_equal(dev.score(0, 6, 6), want)
    assert dev.build_tiles()
    assert np.array_equal(dev.score(0, 6, 6), want)


def test_training_kernel_gives_up_instead_of_hanging(tune):
    """The one-launch training kernel waits for the other workgroups with a
    bounded number of polls.  GTM_FIT_SPIN_LIMIT=abort makes every workgroup give up at
    its first wait whatever it reads there (no dependence on timing or on the number of
    workgroups): the kernel must still drain, the call must report it, and the model must
    be left as it was before the call."""
    from tests.gpu_harness import Device
    from graphtsetlinmachine_amd import _abi

    shape = TILE_SHAPES[3]
    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"], T=30)
    model = helpers.random_model(shape["seed"], cfg, 1, s=3.0, include_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    Y = o.encode_labels(np.zeros(graphs.number_of_graphs, dtype=np.int64), cfg.classes, cfg.threshold)
    tune("GTM_FIT_SPIN_LIMIT", "abort")
    with pytest.raises(_abi.GtmError, match="gave up waiting.*as it was before the call"):
        dev.fit(Y, 0, graphs.number_of_graphs, 0)
    tune("GTM_FIT_SPIN_LIMIT", None)
    ta, _, w = dev.download()
    assert np.array_equal(w, model.clause_weights) and np.array_equal(ta, model.ta_state)
    # the same model trains normally afterwards
    o.fit(model, graphs, Y)
    dev.fit(Y, 0, graphs.number_of_graphs, 0)
    ta, _, w = dev.download()
    assert np.array_equal(w, model.clause_weights) and np.array_equal(ta, model.ta_state)
    # a limit of 0 polls: whoever does not see every arrival at its first look gives up
    tune("GTM_FIT_SPIN_LIMIT", "0")
    try:
        dev.fit(Y, 0, graphs.number_of_graphs, graphs.number_of_graphs)
        o.fit(model, graphs, Y)  # nobody had to wait: the run went through
    except _abi.GtmError as e:
        assert "gave up waiting" in str(e)
    tune("GTM_FIT_SPIN_LIMIT", None)
    ta, _, w = dev.download()
    assert np.array_equal(w, model.clause_weights) and np.array_equal(ta, model.ta_state)


def test_tiles_built_for_another_configuration_are_refused():
    """The driver loops recompute the tile geometry from their arguments; a buffer built for other
    arguments would be read with the wrong row width."""
    from tests.gpu_harness import Device
    from graphtsetlinmachine_amd import _abi

    shape = TILE_SHAPES[3]
    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"], T=30)
    model = helpers.random_model(shape["seed"], cfg, 1, s=3.0, include_density=0.02)
    dev = Device(model, graphs)
    assert dev.build_tiles()
    want = o.score(model, graphs)
    assert np.array_equal(dev.score(0, graphs.number_of_graphs, 8), want)
    # the same buffer handed to a model with message layers (other rows per tile)
    deep_cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"], T=30, depth=2,
                                     message_size=4096)
    deep = Device(helpers.random_model(shape["seed"], deep_cfg, 2), graphs)
    deep.dg.desc.tiles = dev.tiles.data_ptr()
    geometry_differs = _abi.lib.gtm_tiles_bytes(ctypes.byref(deep.acfg), ctypes.byref(deep.dg.desc)) != dev.tiles.numel() * 4
    if geometry_differs:
        with pytest.raises(_abi.GtmError, match="another configuration"):
            deep.score(0, graphs.number_of_graphs, 8)
    # a buffer the library never filled
    import torch

    stray = torch.zeros(dev.tiles.numel(), dtype=torch.int32, device="cuda")
    dev.dg.desc.tiles = stray.data_ptr()
    with pytest.raises(_abi.GtmError, match="not filled by gtm_build_tiles"):
        dev.score(0, graphs.number_of_graphs, 8)
    dev.dg.desc.tiles = dev.tiles.data_ptr()
    assert np.array_equal(dev.score(0, graphs.number_of_graphs, 8), want)


HALF_TILE_SHAPES = [
    # 4, 8, 12, 16 literal words per node; one word per graph up to 64; one to three node types
    dict(seed=51, g=dict(n_graphs=90, max_nodes=31, min_nodes=17, hv_size=64), classes=10, clauses=200, half=False),
    dict(seed=52, g=dict(n_graphs=47, max_nodes=361, min_nodes=300, hv_size=128, max_degree=0), classes=10, clauses=150),
    dict(seed=53, g=dict(n_graphs=45, max_nodes=100, min_nodes=20, hv_size=192, n_symbols=12), classes=3, clauses=90),
    dict(seed=54, g=dict(n_graphs=60, max_nodes=50, min_nodes=17, hv_size=256, n_symbols=12, node_types=("a", "b")),
         classes=4, clauses=64),
    dict(seed=55, g=dict(n_graphs=7, max_nodes=2048, min_nodes=1500, hv_size=64, max_degree=0, node_types=("a", "b", "c")),
         classes=2, clauses=40, half=False),
    # more (graph, class) pairs per tile than four per lane
    dict(seed=56, g=dict(n_graphs=30, max_nodes=361, min_nodes=200, hv_size=128, n_symbols=20, max_degree=0), classes=70,
         clauses=50),
    # so few clauses that the launch which compiles them has fewer workgroups than the tiles have shares
    dict(seed=57, g=dict(n_graphs=50, max_nodes=361, min_nodes=250, hv_size=128, max_degree=0), classes=5, clauses=12),
]


@pytest.mark.parametrize("shape", HALF_TILE_SHAPES, ids=lambda s: "half%d" % s["seed"])
@pytest.mark.parametrize("density", [0.0, 0.02, 0.2])
def test_half_tile_scoring_equals_oracle(shape, density, tune):
    """Depth-1 gtm_score on tiles whose LDS copy holds the positive literals' rows only (negated
    literals as complements; data declared complementary after the library's own check) == oracle
    == the bitmap path == the tiles of all rows."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"])
    model = helpers.random_model(shape["seed"], cfg, 1, include_density=density)
    top = cfg.state_bits - 1
    model.ta_state[3, :, top] = 0  # an empty clause among the random ones
    rng = np.random.default_rng(shape["seed"])
    used = np.unique(graphs.hypervectors)
    hv = graphs.hypervector_size
    # clauses of positive literals only, of negated literals only (each holds at nearly every node), of one
    # literal, of exactly 7 + 7 (one of the 14 rarest is left to phase 2), and with x and NOT x together
    def include(c, literals):
        model.ta_state[c, :, top] = 0
        for l in literals:
            model.ta_state[c, l // 32, top] |= np.uint32(1 << (l % 32))
    include(4, rng.choice(used, size=min(5, used.size), replace=False))
    include(5, hv + rng.choice(hv, size=30, replace=False))
    include(6, [int(used[0])])
    include(7, [hv + int(used[0])])
    include(8, list(rng.choice(used, size=min(7, used.size), replace=False)) + list(hv + rng.choice(hv, size=7, replace=False)))
    include(9, [int(used[1]), hv + int(used[1])])
    include(10, hv + rng.choice(hv, size=3, replace=False))
    include(11, list(rng.choice(used, size=min(3, used.size), replace=False)) + list(hv + rng.choice(hv, size=2, replace=False)))
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    plain = dev.score(0, G, G)
    assert dev.build_tiles()
    full = dev.score(0, G, G)
    assert dev.declare_complementary()
    assert dev.build_tiles()
    _abi.call("gtm_profile_enable", 1)
    half = dev.score(0, G, G)
    name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
    _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
    _abi.call("gtm_profile_enable", 0)
    # the half tiles are taken where they hold more graphs than the tiles of all rows
    expected = "k_tile_two_phase_half<score>" if shape.get("half", True) else "k_tile_two_phase<score>"
    assert name.value.decode() == expected
    assert np.array_equal(full, plain) and np.array_equal(half, plain)
    sample = sorted(set([0, 1, G // 2, G - 1]))
    assert np.array_equal(half[sample], o.score(model, graphs, sample))
    assert np.array_equal(dev.score(3, G - 5, G), plain[3:G - 2])  # a range that starts and ends inside tiles
    if shape.get("half", True):
        # fewer workgroups than tiles, the tiles' clauses shared out evenly among them (what a launch does whose
        # tiles do not fill a whole number of rounds of the chip): a workgroup takes the end of one tile's clauses,
        # whole tiles and the start of another's, and workgroups that share a tile add their class sums
        for groups in (1, 2, 3, 5):
            tune("GTM_TILE_LINE_GROUPS", str(groups))
            assert np.array_equal(dev.score(0, G, G), plain), groups
            assert np.array_equal(dev.score(3, G - 5, G), plain[3:G - 2]), groups
        tune("GTM_TILE_LINE_GROUPS", None)
    # one-launch training on the same tiles follows the oracle
    Y = o.encode_labels(rng.integers(0, cfg.classes, size=G), cfg.classes, cfg.threshold)
    o.fit(model, graphs, Y)
    dev.fit(Y, 0, G, 0)
    ta, _, w = dev.download()
    assert np.array_equal(w, model.clause_weights) and np.array_equal(ta, model.ta_state)
    assert np.array_equal(dev.score(0, G, G)[sample], o.score(model, graphs, sample))


def test_data_that_is_not_complementary_is_detected_and_keeps_all_rows():
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(57, n_graphs=20, max_nodes=60, min_nodes=20, hv_size=64)
    cfg = helpers.oracle_config(graphs, classes=3, clauses=40)
    model = helpers.random_model(57, cfg, 1, include_density=0.03)
    assert Device(model, graphs).properties() == (0, 0)
    # a node whose literal 5 and its negation are both set (X is a public array: a user can do this)
    broken = copy.deepcopy(graphs)
    row = int(broken.node_index[7]) + 3
    broken.X[row, 0] |= np.uint32(1 << 5)
    broken.X[row, 2] |= np.uint32(1 << 5)
    dev = Device(model, broken)
    assert dev.properties() == (1, 0) and not dev.declare_complementary()
    assert dev.build_tiles()
    assert np.array_equal(dev.score(0, 20, 20), o.score(model, broken))
    # a graph without nodes rules the half tiles out as well
    sizes = [30, 0, 40, 25]
    empty = helpers.random_graphs(58, n_graphs=4, hv_size=64, sizes=sizes)
    dev = Device(model, empty)
    assert dev.properties() == (0, 1) and not dev.declare_complementary()
    # a width of the literal halves that is not a multiple of 32 is compared bit by bit
    odd = helpers.random_graphs(59, n_graphs=6, max_nodes=20, hv_size=20)
    odd_cfg = helpers.oracle_config(odd, classes=2, clauses=10)
    dev = Device(helpers.random_model(59, odd_cfg, 1), odd)
    assert dev.properties() == (0, 0)
    odd.X[2, 1] ^= np.uint32(1 << 3)  # literal 35 = the negation of literal 15
    assert Device(helpers.random_model(59, odd_cfg, 1), odd).properties() == (1, 0)


@pytest.mark.parametrize("shape", [s for s in TILE_SHAPES if s["seed"] in (14, 15, 16, 17, 18)], ids=lambda s: "tiles%d" % s["seed"])
def test_the_kernel_that_takes_over_beyond_4_gib_of_literal_words_follows_the_oracle(shape, tune):
    """k_tile_two_phase addresses X with 32-bit byte offsets and hands data sets of 4 GiB and more to
    k_tile_two_phase_wide (64-bit offsets).  GTM_NO_NARROW_TWO_PHASE takes that way with small data."""
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(shape["seed"], **shape["g"])
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=shape["clauses"])
    model = helpers.random_model(shape["seed"], cfg, 1, include_density=0.05)
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    assert dev.build_tiles()
    tune("GTM_NO_NARROW_TWO_PHASE", "1")
    _abi.call("gtm_profile_enable", 1)
    got = dev.score(0, G, G)
    name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
    _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
    _abi.call("gtm_profile_enable", 0)
    assert name.value.decode() == "k_tile_two_phase_wide<score>"
    assert np.array_equal(got, o.score(model, graphs))


NARROW_TILE_SHAPES = [
    # one graph of 22 truth words per tile (the message rows leave room for no more); three graphs of 10 words
    # per tile; the same with a graph without nodes (then the data set is not declared complementary: layer 0
    # takes the kernels that keep every row, the message layers scan every clause); several node types
    dict(seed=61, g=dict(n_graphs=5, sizes=[700, 520, 1, 33, 689], hv_size=64, edge_types=("l", "r")), classes=3),
    dict(seed=62, g=dict(n_graphs=11, max_nodes=300, min_nodes=1, hv_size=64, edge_types=("l", "r", "u")), classes=2),
    dict(seed=63, g=dict(n_graphs=7, sizes=[300, 0, 1, 290, 0, 17, 64], hv_size=64, edge_types=("l",)), classes=4),
    dict(seed=64, g=dict(n_graphs=6, max_nodes=650, min_nodes=400, hv_size=352, n_symbols=9, node_types=("a", "b", "c"),
                         edge_types=("l", "r")), classes=3),
    # rows of 33 to 64 words (messages of 512 bits, so that their rows fit beside them): one graph of up to 2,000
    # nodes per tile; two graphs of 32 words per tile, one of them without nodes in one tile
    dict(seed=65, g=dict(n_graphs=4, sizes=[1500, 1025, 2000, 33], hv_size=64, edge_types=("l", "r")), classes=3, M=512),
    dict(seed=66, g=dict(n_graphs=6, sizes=[1000, 900, 0, 1000, 512, 1], hv_size=64, edge_types=("l", "r", "u")), classes=2,
         M=512),
]


@pytest.mark.parametrize("shape", NARROW_TILE_SHAPES, ids=lambda s: "narrow%d" % s["seed"])
@pytest.mark.parametrize("depth", [1, 2, 3])
@pytest.mark.parametrize("path", ["several-clauses-per-wave", "128-bit-reads", "rows-as-stored", "clauses-by-number", "all-rows-layer-0",
                                  "one-clause-per-wave", "messages-of-a-tile-in-lds", "messages-in-three-launches"])
def test_scoring_on_narrow_tiles(shape, depth, path, tune):
    """Tiles whose rows are at most 64 words wide: eight or four clauses per wave (score_narrow.h), for the message
    layers and - on a data set whose negated literals are the complements of its positive ones - for
    layer 0 on the positive rows alone; against the oracle and against the kernels that take one clause
    per wave.  The clauses are of three kinds: random ones (most die within the first rows), ones made of
    a few hundred literals that hold everywhere (negations of hypervector and message bits that nothing
    sets: their lists take several windows of 128 entries and are walked to the end), and empty ones."""
    from tests.gpu_harness import Device

    if path == "128-bit-reads":  # (rows of at most 32 words: eight clauses per wave, four words per lane)
        tune("GTM_NARROW_READS", "128")
    elif path == "rows-as-stored":  # (rows in LDS as far apart as in memory, not 128 bytes)
        tune("GTM_NARROW_ROWS_AS_STORED", "1")
    elif path == "clauses-by-number":  # (layer 0 takes clauses q, q + streams, ... instead of by length of their lists)
        tune("GTM_NARROW_IN_ORDER", "1")
    elif path == "all-rows-layer-0":
        tune("GTM_NO_HALF_ROWS", "1")
    elif path == "one-clause-per-wave":
        tune("GTM_NO_NARROW_LAYERS", "1")
    elif depth == 1:
        pytest.skip("no messages at depth 1")
    elif path == "messages-of-a-tile-in-lds":  # (score_messages.h; by itself only where a graph's vectors are too big
        tune("GTM_MESSAGES_IN_LDS", "1")       # for one workgroup per graph: the graphs of 650 and 700 nodes here)
    elif path == "messages-in-three-launches":
        tune("GTM_MESSAGES_IN_LDS", "0")
        tune("GTM_NO_FUSED_MESSAGES", "1")
    graphs = helpers.random_graphs(shape["seed"], max_degree=3, **shape["g"])
    hv = graphs.hypervector_size
    M = shape.get("M", 1024) if depth > 1 else 64
    cfg = helpers.oracle_config(graphs, classes=shape["classes"], clauses=150, depth=depth, message_size=M)
    # (random clauses of about three literals: some are true at some nodes of some graphs)
    model = helpers.random_model(shape["seed"], cfg, depth, include_density=1.5 / hv, message_density=0.004)
    rng = np.random.default_rng(shape["seed"])
    top = cfg.state_bits - 1
    unused = np.setdiff1d(np.arange(hv), np.unique(graphs.hypervectors))
    sent = np.unique((model.hypervectors.reshape(-1, 1) + np.arange(4).reshape(1, -1)) % M)  # bits a message can hold
    unsent = np.setdiff1d(np.arange(M), sent)
    for c in range(0, cfg.clauses, 3):  # every third clause holds wherever its node type is
        model.ta_state[c, :, top] = 0
        for k in rng.permutation(unused)[: int(rng.integers(0, len(unused) + 1))]:
            lit = hv + int(k)
            model.ta_state[c, lit // 32, top] |= np.uint32(1 << (lit % 32))
        for bank in model.message_ta_state:
            bank[c, :, top] = 0
            for p in rng.permutation(unsent)[: int(rng.integers(0, 500))]:
                lit = M + int(p)
                bank[c, lit // 32, top] |= np.uint32(1 << (lit % 32))
    model.ta_state[6, :, top] = 0  # an empty clause
    dev = Device(model, graphs)
    G = graphs.number_of_graphs
    want = o.score(model, graphs)
    assert want.any()
    complementary = dev.declare_complementary()
    assert complementary == (0 not in list(shape["g"].get("sizes", [1])))
    assert dev.build_tiles(), "this shape should have a tile layout"
    assert np.array_equal(dev.score(0, G, G), want)
    assert np.array_equal(dev.score(0, G, 2), want)       # several launch groups
    if G > 5:
        assert np.array_equal(dev.score(2, G - 3, 4), want[2:G - 1])  # a range that starts and ends inside tiles
