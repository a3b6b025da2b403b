"""The public model API on the GPU against the oracle driven the same way."""

import numpy as np
import pytest

from graphtsetlinmachine_amd import workloads
from oracle import gtm_oracle as o
from tests import helpers

pytestmark = pytest.mark.gpu


def oracle_twin(tm, graphs):
    cfg = o.Config(classes=tm.number_of_outputs, clauses=tm.number_of_clauses, literals=tm.number_of_literals,
                   state_bits=tm.number_of_state_bits, boost_true_positive_feedback=tm.boost_true_positive_feedback,
                   threshold=tm.T, q=tm.q, max_included_literals=tm.max_included_literals,
                   max_nodes=int(graphs.max_number_of_graph_nodes), message_size=tm.message_size,
                   message_bits=tm.message_bits)
    return o.new_model(cfg, tm.depth, tm.s, tm.hypervectors, seed=tm.seed)


def assert_same_state(tm, model):
    state = tm.save()
    assert np.array_equal(state["ta_state"], model.ta_state.reshape(-1))
    assert np.array_equal(state["clause_weights"].reshape(model.clause_weights.shape), model.clause_weights)
    for got, want in zip(state["message_ta_state"], model.message_ta_state):
        assert np.array_equal(got, want.reshape(-1))


def test_noisy_xor_end_to_end_matches_oracle_and_learns():
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.noisy_xor(1500, 500)
    np.random.seed(3)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=99)
    model = None
    for epoch in range(2):
        tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
        if model is None:
            model = oracle_twin(tm, wl.graphs_train)
        o.fit(model, wl.graphs_train, o.encode_labels(wl.Y_train, 2, tm.T))
        assert_same_state(tm, model)
    sums = tm.score(wl.graphs_test)
    assert np.array_equal(sums, o.score(model, wl.graphs_test))
    assert np.array_equal(tm.predict(wl.graphs_test), sums.argmax(axis=1))
    assert (tm.predict(wl.graphs_test) == wl.Y_test).mean() == 1.0
    assert (tm.predict(wl.graphs_train) == wl.Y_train).mean() >= 0.975
    # introspection used by every demo's tail
    assert tm.get_weights().shape == (2, 10)
    plane = model.ta_state[:, :, 7]
    for clause in (0, 9):
        for ta in (0, 17, 33, 63):
            assert bool(tm.ta_action(0, clause, ta)) == bool((plane[clause, ta // 32] >> (ta % 32)) & 1)
    assert tm.get_state()[2:8] == (2, 10, 64, 2, 8, 2)


def test_the_readme_sequence_task_is_learned_through_three_layers():
    """README.md:194-208 / examples/SequenceClassificationDemo.py: one run of 1, 2 or 3 'A's in a
    chain with 'Left'/'Right' edges.  Single nodes cannot tell the classes apart, so 100 % on
    clean test data needs messages, their rotation by edge type and the feedback of all three
    banks to work together.  The oracle, handed the final state, scores a sample of the test
    graphs."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.runs_of_a(12000, 3000)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=7)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=2, incremental=True)
    assert (tm.predict(wl.graphs_test) == wl.Y_test).mean() >= 0.99
    assert (tm.predict(wl.graphs_train) == wl.Y_train).mean() >= 0.97  # 1 % of the training labels are wrong
    trained = oracle_twin(tm, wl.graphs_train)
    state = tm.get_state()
    cfg = trained.cfg
    trained.ta_state = state[0].reshape(cfg.clauses, cfg.la_chunks, cfg.state_bits).copy()
    trained.message_ta_state = [b.reshape(cfg.clauses, cfg.message_chunks, cfg.state_bits).copy()
                                for b in tm.message_ta_state]
    trained.clause_weights = state[1].reshape(cfg.classes, cfg.clauses).copy()
    sample = list(range(40))
    assert np.array_equal(tm.score(wl.graphs_test)[sample], o.score(trained, wl.graphs_test, sample))


def test_save_load_roundtrip_and_resume(tmp_path):
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.noisy_xor(300, 100)
    np.random.seed(4)
    a = MultiClassGraphTsetlinMachine(**wl.params, seed=5)
    a.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    path = str(tmp_path / "model.pkl")
    state = a.save(path, format="pickle")  # the reference's file format (tm.py:356-357)
    reference_keys = {
        "ta_state", "message_ta_state", "clause_weights", "hypervectors", "number_of_outputs", "number_of_literals",
        "number_of_message_literals", "min_y", "max_y", "negative_clauses", "max_number_of_graph_nodes",
        "number_of_clauses", "T", "s", "q", "max_included_literals", "boost_true_positive_feedback",
        "number_of_state_bits", "depth", "message_size", "message_bits", "double_hashing", "one_hot_encoding",
    }
    assert reference_keys <= set(state)
    assert state["ta_state"].dtype == np.uint32 and state["ta_state"].shape == (10 * 2 * 8,)
    assert state["clause_weights"].dtype == np.int32
    b = MultiClassGraphTsetlinMachine(**wl.params, seed=777)
    b.load(fname=path)
    assert np.array_equal(b.score(wl.graphs_test), a.score(wl.graphs_test))
    # by default the file is an archive of plain arrays whatever it is called; load tells by the content
    plain = str(tmp_path / "model.tm")
    a.save(plain)
    with np.load(plain, allow_pickle=False) as z:
        assert "ta_state" in z.files
    c = MultiClassGraphTsetlinMachine(**wl.params, seed=778)
    c.load(fname=plain)
    assert np.array_equal(c.score(wl.graphs_test), a.score(wl.graphs_test))
    # resuming from the file continues exactly where the first model would have gone
    a.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    b.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    sa, sb = a.save(), b.save()
    assert np.array_equal(sa["ta_state"], sb["ta_state"]) and np.array_equal(sa["clause_weights"], sb["clause_weights"])
    assert np.array_equal(sa["message_ta_state"][0], sb["message_ta_state"][0])


def test_ragged_multi_type_graphs_depth3_match_oracle():
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    train = helpers.random_graphs(50, n_graphs=40, max_nodes=45, hv_size=24, node_types=("a", "b"),
                                  edge_types=("l", "r", "u"), max_degree=3)
    test = helpers.random_graphs(51, n_graphs=25, max_nodes=60, parent=train, node_types=("a", "b"),
                                 edge_types=("l", "r", "u"), max_degree=3)  # larger graphs than seen in training
    rng = np.random.default_rng(1)
    Y = rng.integers(0, 3, size=40)
    np.random.seed(8)
    tm = MultiClassGraphTsetlinMachine(60, 40, (2.0, 1.5, 3.0), depth=3, message_size=48, message_bits=2,
                                       max_included_literals=12, seed=2024)
    tm.fit(train, Y, epochs=2, incremental=True)
    model = oracle_twin(tm, train)
    o.fit(model, train, o.encode_labels(Y, 3, tm.T), epochs=2)
    assert_same_state(tm, model)
    model.cfg = oracle_twin(tm, test).cfg  # bitmap stride follows the scored data set
    assert np.array_equal(tm.score(test), o.score(model, test))


def test_fit_not_incremental_resets_layer_zero_only():
    """tm.py:524-526: a second fit(incremental=False) re-runs `prepare` only."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.noisy_xor(200, 50)
    np.random.seed(6)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=11)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1)
    before = tm.save()
    tm.fit(wl.graphs_train, wl.Y_train, epochs=0)
    after = tm.save()
    fresh = o.prepare(oracle_twin(tm, wl.graphs_train).cfg, 11, tm.step)
    assert np.array_equal(after["ta_state"], fresh[0].reshape(-1))
    assert np.array_equal(after["clause_weights"].reshape(2, -1), fresh[1])
    assert np.array_equal(after["message_ta_state"][0], before["message_ta_state"][0])


def test_score_before_fit_exits_like_the_reference():
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.noisy_xor(10, 10)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=1)
    with pytest.raises(SystemExit):
        tm.score(wl.graphs_test)


def test_transform_and_read_outs_match_the_oracle():
    """transform / transform_nodewise / get_ta_states / get_hyperliterals (bit-exact against the
    oracle) and the two host read-outs built on them (against a literal-level recount)."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    train = helpers.random_graphs(60, n_graphs=30, hv_size=24, node_types=("a", "b"), edge_types=("l", "r"),
                                  sizes=[5, 0, 33, 1, 40, 64] * 5)
    rng = np.random.default_rng(2)
    Y = rng.integers(0, 3, size=30)
    np.random.seed(9)
    tm = MultiClassGraphTsetlinMachine(40, 30, (2.0, 1.5), depth=2, message_size=40, message_bits=2, seed=11)
    tm.fit(train, Y, epochs=2, incremental=True)
    model = oracle_twin(tm, train)
    o.fit(model, train, o.encode_labels(Y, 3, tm.T), epochs=2)
    assert_same_state(tm, model)

    got, sums = tm.transform(train)
    want, want_sums = o.transform(model, train)
    assert got.dtype == np.int32 and np.array_equal(got, want) and np.array_equal(sums, want_sums)
    assert got.any() and not got[1].any()  # a graph without nodes transforms to zeros
    wide, sums = tm.transform_nodewise(train)
    want, _ = o.transform(model, train, nodewise=True)
    assert wide.shape == (30, 40, 64) and np.array_equal(wide, want) and np.array_equal(sums, want_sums)

    for depth, bank, literals in ((0, model.ta_state, tm.number_of_literals),
                                  (1, model.message_ta_state[0], tm.number_of_message_literals)):
        assert np.array_equal(tm.get_ta_states(depth), o.get_ta_states(bank, 8, literals))
        assert np.array_equal(tm.get_hyperliterals(depth), o.get_hyperliterals(bank, 8, literals))

    # get_clause_literals: per clause and symbol, the number of the symbol's bits among the included literals
    included = o.get_hyperliterals(model.ta_state, 8, tm.number_of_literals)
    table = tm.get_clause_literals(train.hypervectors)
    n_symbols, half = train.hypervectors.shape[0], tm.number_of_literals // 2
    assert table.shape == (40, 2 * n_symbols)
    for c in (0, 7, 39):
        for sym in range(n_symbols):
            bits = [int(b) for b in train.hypervectors[sym]]
            assert table[c, sym] == sum(int(included[c, b]) for b in bits)
            assert table[c, n_symbols + sym] == sum(int(included[c, half + b]) for b in bits)
    # get_messages: the same count for the sending clauses' hypervector bits rotated by the edge type
    included = o.get_hyperliterals(model.message_ta_state[0], 8, tm.number_of_message_literals)
    messages = tm.get_messages(1, 2)
    assert messages.shape == (2, 40, 80)
    for edge_type in (0, 1):
        for c in (0, 13):
            for sender in (0, 5, 39):
                bits = [(int(b) + edge_type) % 40 for b in tm.hypervectors[sender]]
                assert messages[edge_type, c, sender] == sum(int(included[c, b]) for b in bits)
                assert messages[edge_type, c, 40 + sender] == sum(int(included[c, 40 + b]) for b in bits)


@pytest.mark.parametrize("case", [
    # 361-node graphs, one layer (tiles of positive rows only); tiny graphs that share words of a tile row;
    # two and three layers with edge types and graphs without nodes; one graph of 21 words per tile (four
    # clauses per wave)
    dict(g=dict(n_graphs=23, max_nodes=361, min_nodes=300, hv_size=128), m=dict(depth=1), clauses=70, classes=10),
    dict(g=dict(n_graphs=90, max_nodes=3, hv_size=16, node_types=("a", "b")), m=dict(depth=1), clauses=33, classes=2),
    dict(g=dict(n_graphs=30, hv_size=24, node_types=("a", "b"), edge_types=("l", "r"), sizes=[5, 0, 33, 1, 40, 64] * 5),
         m=dict(depth=2, message_size=64, message_bits=2), clauses=40, classes=3),
    dict(g=dict(n_graphs=20, max_nodes=20, min_nodes=4, hv_size=20, edge_types=("x", "y", "z")),
         m=dict(depth=3, message_size=37, message_bits=3), clauses=50, classes=4),
    dict(g=dict(n_graphs=6, max_nodes=650, min_nodes=400, hv_size=64, edge_types=("l", "r")),
         m=dict(depth=3, message_size=1024, message_bits=2), clauses=60, classes=3),
], ids=["361-nodes", "tiny-graphs", "two-layers", "three-layers", "narrow-tiles"])
def test_transform_on_tiles(case, tune):
    """gtm_transform from the truth rows of the tile kernels (k_tile_transform) == the dense path ==
    the oracle: per-clause outputs, per-node outputs and class sums, in one launch group and in groups
    of 7 graphs (which start and end inside tiles)."""
    import ctypes
    from graphtsetlinmachine_amd import _abi
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    graphs = helpers.random_graphs(77, **case["g"])
    n = graphs.number_of_graphs
    depth = case["m"]["depth"]
    rng = np.random.default_rng(3)
    Y = rng.integers(0, case["classes"], size=n)
    np.random.seed(5)
    tm = MultiClassGraphTsetlinMachine(case["clauses"], 30, (2.0, 1.5, 1.2)[:depth] if depth > 1 else 2.0, seed=13, **case["m"])
    tm.fit(graphs, Y, epochs=2, incremental=True)
    model = oracle_twin(tm, graphs)  # an untrained oracle model of the same shape, given the trained state
    state = tm.save()
    model.ta_state = state["ta_state"].reshape(model.ta_state.shape).copy()
    model.clause_weights = state["clause_weights"].reshape(model.clause_weights.shape).copy()
    model.message_ta_state = [bank.reshape(init.shape).copy() for bank, init in zip(state["message_ta_state"], model.message_ta_state)]
    want, want_sums = o.transform(model, graphs)
    want_wide, _ = o.transform(model, graphs, nodewise=True)
    assert want.any() and not want.all()

    name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
    _abi.call("gtm_profile_enable", 1)
    got, sums = tm._transform(graphs, False)
    _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
    _abi.call("gtm_profile_enable", 0)
    assert name.value == b"k_tile_transform", "the tile path should have run"
    assert np.array_equal(got, want) and np.array_equal(sums, want_sums)
    assert np.array_equal(sums, tm.score_device(graphs).cpu().numpy().reshape(n, -1))
    wide, sums = tm._transform(graphs, True, batch=7)
    assert np.array_equal(wide, want_wide) and np.array_equal(sums, want_sums)
    got, sums = tm._transform(graphs, False, batch=7)
    assert np.array_equal(got, want) and np.array_equal(sums, want_sums)
    tune("GTM_NO_TILE_TRANSFORM", "1")
    dense, dense_sums = tm._transform(graphs, False)
    assert np.array_equal(dense, want) and np.array_equal(dense_sums, want_sums)


def test_multi_output_and_single_output_heads_follow_the_oracle():
    """tm.py:961-1072: several independent outputs (Y in {0, 1} per output, prediction sum >= 0) and
    the single-output machine (one 'class', score is a vector): states, sums and predictions."""
    from graphtsetlinmachine_amd.tm import GraphTsetlinMachine, MultiOutputGraphTsetlinMachine

    wl = workloads.noisy_xor(1200, 300)
    x_train = wl.Y_train.astype(np.int64)
    Y3 = np.stack([x_train, 1 - x_train, np.ones_like(x_train)], axis=1)
    params = dict(wl.params)
    tm = MultiOutputGraphTsetlinMachine(**params, seed=5)
    tm.fit(wl.graphs_train, Y3, epochs=0, incremental=True)
    model = oracle_twin(tm, wl.graphs_train)
    assert model.cfg.classes == 3
    tm.fit(wl.graphs_train, Y3, epochs=2, incremental=True)
    o.fit(model, wl.graphs_train, np.where(Y3 == 1, tm.T, -tm.T).astype(np.int32), epochs=2)
    assert_same_state(tm, model)
    sums = tm.score(wl.graphs_test)
    assert np.array_equal(sums, o.score(model, wl.graphs_test))
    pred = tm.predict(wl.graphs_test)
    assert pred.dtype == np.uint32 and np.array_equal(pred, (sums >= 0).astype(np.uint32))
    assert (pred[:, 0] == wl.Y_test).mean() == 1.0 and (pred[:, 1] == 1 - wl.Y_test).mean() == 1.0 and pred[:, 2].all()

    one = GraphTsetlinMachine(**params, seed=6)
    one.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)
    model = oracle_twin(one, wl.graphs_train)
    assert model.cfg.classes == 1
    one.fit(wl.graphs_train, wl.Y_train, epochs=2, incremental=True)
    o.fit(model, wl.graphs_train, np.where(wl.Y_train == 1, one.T, -one.T).astype(np.int32).reshape(-1, 1), epochs=2)
    assert_same_state(one, model)
    score = one.score(wl.graphs_test)
    assert score.shape == (300,) and np.array_equal(score, o.score(model, wl.graphs_test)[:, 0])
    assert np.array_equal(one.predict(wl.graphs_test), score >= 0)
    assert (one.predict(wl.graphs_test) == (wl.Y_test == 1)).mean() == 1.0


def test_the_call_sequence_of_the_noisy_xor_demo_runs_unchanged():
    """A user's script written against the reference (the calls and attributes of
    examples/NoisyXORDemo.py: per-call graph building, `init_with`, grid/block arguments, one
    epoch per fit call, the clause read-out loop at the end) works with the import swapped."""
    from graphtsetlinmachine_amd.graphs import Graphs
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    rng = np.random.default_rng(3)
    np.random.seed(3)

    def build(n, init_with=None, noise=0.0):
        if init_with is None:
            graphs = Graphs(n, symbols=["A", "B"], hypervector_size=32, hypervector_bits=2)
        else:
            graphs = Graphs(n, init_with=init_with)
        for graph_id in range(n):
            graphs.set_number_of_graph_nodes(graph_id, 2)
        graphs.prepare_node_configuration()
        for graph_id in range(n):
            graphs.add_graph_node(graph_id, "Node 1", 1)
            graphs.add_graph_node(graph_id, "Node 2", 1)
        graphs.prepare_edge_configuration()
        Y = np.empty(n, dtype=np.uint32)
        for graph_id in range(n):
            graphs.add_graph_node_edge(graph_id, "Node 1", "Node 2", "Plain")
            graphs.add_graph_node_edge(graph_id, "Node 2", "Node 1", "Plain")
            x1, x2 = rng.integers(0, 2, size=2)
            graphs.add_graph_node_property(graph_id, "Node 1", "A" if x1 else "B")
            graphs.add_graph_node_property(graph_id, "Node 2", "A" if x2 else "B")
            Y[graph_id] = x1 ^ x2
            if rng.random() <= noise:
                Y[graph_id] = 1 - Y[graph_id]
        graphs.encode()
        return graphs, Y

    graphs_train, Y_train = build(2000, noise=0.01)
    graphs_test, Y_test = build(500, init_with=graphs_train)
    assert graphs_test.hypervectors is graphs_train.hypervectors or np.array_equal(graphs_test.hypervectors,
                                                                                  graphs_train.hypervectors)
    assert graphs_train.signature != graphs_test.signature and len(graphs_train) == 2000

    # (the demo's default limit of 4 included literals makes learning depend on the seed, in the CPU
    # oracle as well: the limit is left at its constructor default here)
    tm = MultiClassGraphTsetlinMachine(10, 100, 1.0, depth=2, message_size=256, message_bits=2,
                                       max_included_literals=None, grid=(16 * 13, 1, 1), block=(128, 1, 1))
    for _ in range(3):
        tm.fit(graphs_train, Y_train, epochs=1, incremental=True)
        result_test = 100 * (tm.predict(graphs_test) == Y_test).mean()
        result_train = 100 * (tm.predict(graphs_train) == Y_train).mean()
    assert result_test == 100.0 and result_train >= 97.0

    weights = tm.get_state()[1].reshape(2, -1)
    assert weights.shape == (2, tm.number_of_clauses)
    described = []
    for i in range(tm.number_of_clauses):
        literals = []
        for k in range(graphs_train.hypervector_size * 2):
            if tm.ta_action(0, i, k):
                literals.append(("x%d" if k < graphs_train.hypervector_size else "NOT x%d")
                                % (k % graphs_train.hypervector_size))
        for k in range(tm.message_size * 2):
            if tm.ta_action(1, i, k):
                literals.append(("c%d" if k < tm.message_size else "NOT c%d") % (k % tm.message_size))
        described.append(" AND ".join(literals))
    assert any(described) and tm.hypervectors.shape == (10, 2)
    assert graphs_train.edge_type_id == {"Plain": 0} and set(graphs_train.symbol_id) == {"A", "B"}


@pytest.mark.parametrize("encoding, clauses, edge_types, depth", [
    ("one_hot_encoding", 30, ("l", "r", "u"), 2),     # message size 90: not a multiple of 32
    ("one_hot_encoding", 32, ("l", "r"), 3),          # message size 64: the factored message kernels
    ("one_hot_encoding", 12, ("l",), 2),
    ("double_hashing", 40, ("l", "r", "u"), 3),
    ("double_hashing", 70, ("l", "r"), 2),   # more clauses than message bits: hypervectors repeat
])
def test_one_hot_and_double_hashed_clause_messages_follow_the_oracle(encoding, clauses, edge_types, depth):
    """tm.py:90-106,415-418: the two deterministic clause hypervector tables.  One-hot sizes the
    messages at the first fit (clauses x edge types), after the constructor made the table.
    Training trajectories and class sums are compared with the oracle given the same table."""
    from sympy import prevprime

    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    train = helpers.random_graphs(70, n_graphs=36, max_nodes=50, hv_size=24, node_types=("a", "b"),
                                  edge_types=edge_types, max_degree=3)
    test = helpers.random_graphs(71, n_graphs=20, max_nodes=70, parent=train, node_types=("a", "b"),
                                 edge_types=edge_types, max_degree=3)
    Y = np.random.default_rng(5).integers(0, 3, size=36)
    kwargs = {encoding: True}
    tm = MultiClassGraphTsetlinMachine(clauses, 40, (2.0, 1.5, 3.0)[:depth], depth=depth, message_size=64,
                                       message_bits=3, max_included_literals=14, seed=31, **kwargs)
    tm.fit(train, Y, epochs=2, incremental=True)
    n_types = len(train.edge_type_id)
    if encoding == "one_hot_encoding":
        assert tm.message_size == clauses * n_types and tm.message_bits == 1
        assert np.array_equal(tm.hypervectors[:, 0], np.arange(clauses) * n_types)
    else:
        p = int(prevprime(64))
        ids = np.arange(clauses)
        assert tm.message_size == 64 and tm.message_bits == 2
        assert np.array_equal(tm.hypervectors, np.stack([ids % 64, p - ids % p], axis=1))
    model = oracle_twin(tm, train)
    assert model.cfg.message_size == tm.message_size and model.cfg.message_bits == tm.message_bits
    o.fit(model, train, o.encode_labels(Y, 3, tm.T), epochs=2)
    assert_same_state(tm, model)
    model.cfg = oracle_twin(tm, test).cfg
    assert np.array_equal(tm.score(test), o.score(model, test))
    saved = tm.save()
    assert saved["message_size"] == tm.message_size and saved[encoding] is True
    again = MultiClassGraphTsetlinMachine(clauses, 40, (2.0, 1.5, 3.0)[:depth], depth=depth, **kwargs)
    again.load(saved)
    assert np.array_equal(again.score(test), tm.score(test))


def _reference_dict(state):
    """The dict exactly as the reference's save() writes it: its 23 keys (tm.py:328-354), no generator position."""
    from tests.test_model_host import REFERENCE_KEYS

    return {key: state[key] for key in REFERENCE_KEYS}


def test_a_state_dict_shaped_like_the_references_loads_scores_and_resumes(tmp_path):
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    train = helpers.random_graphs(80, n_graphs=30, max_nodes=40, hv_size=20, edge_types=("l", "r"), max_degree=2)
    Y = np.random.default_rng(6).integers(0, 2, size=30)
    np.random.seed(12)
    a = MultiClassGraphTsetlinMachine(24, 30, (1.5, 2.5), depth=2, message_size=40, message_bits=2, seed=77)
    a.fit(train, Y, epochs=1, incremental=True)
    model = oracle_twin(a, train)
    o.fit(model, train, o.encode_labels(Y, 2, a.T))
    assert_same_state(a, model)
    state = _reference_dict(a.save())
    assert len(state) == 23 and "rng_seed" not in state

    # a model constructed with other arguments takes its shape from the dict
    b = MultiClassGraphTsetlinMachine(5, 7, 9.0, seed=77)
    b.load(state)
    assert (b.number_of_clauses, b.depth, b.T, b.s) == (24, 2, 30, (1.5, 2.5))
    assert np.array_equal(b.score(train), o.score(model, train))
    # resuming: without a generator position the loaded model starts its draws at step 0 of its own seed
    b.fit(train, Y, epochs=1, incremental=True)
    resumed = oracle_twin(b, train)
    resumed.ta_state, resumed.message_ta_state = model.ta_state.copy(), [m.copy() for m in model.message_ta_state]
    resumed.clause_weights = model.clause_weights.copy()
    resumed.step = 0
    o.fit(resumed, train, o.encode_labels(Y, 2, b.T))
    assert_same_state(b, resumed)

    # the archive without pickle: same state, generator position included, so both go on identically
    path = str(tmp_path / "model.npz")
    a.save(path)
    with np.load(path, allow_pickle=False) as z:
        assert "ta_state" in z.files and "message_ta_state_0" in z.files
    c = MultiClassGraphTsetlinMachine(24, 30, (1.5, 2.5), depth=2, message_size=40, message_bits=2, seed=1)
    c.load(fname=path)
    assert c.seed == 77 and c.step == a.step
    assert np.array_equal(c.score(train), a.score(train))
    a.fit(train, Y, epochs=1, incremental=True)
    c.fit(train, Y, epochs=1, incremental=True)
    sa, sc = a.save(), c.save()
    assert np.array_equal(sa["ta_state"], sc["ta_state"]) and np.array_equal(sa["clause_weights"], sc["clause_weights"])
    assert np.array_equal(sa["message_ta_state"][0], sc["message_ta_state"][0])

    # a state whose arrays do not fit its sizes is refused before anything is copied to the device
    bad = dict(state)
    bad["ta_state"] = state["ta_state"][:-1]
    with pytest.raises(Exception, match="ta_state"):
        MultiClassGraphTsetlinMachine(24, 30, 1.0).load(bad)


def test_set_state_builds_a_usable_model_from_a_state_tuple():
    """tm.py:289-310 made functional: on a model that never trained, with message banks."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    train = helpers.random_graphs(81, n_graphs=30, max_nodes=40, hv_size=20, edge_types=("l", "r"), max_degree=2)
    Y = np.random.default_rng(7).integers(0, 3, size=30)
    np.random.seed(13)
    a = MultiClassGraphTsetlinMachine(24, 30, (1.5, 2.5), depth=2, message_size=40, message_bits=2, seed=5)
    a.fit(train, Y, epochs=1, incremental=True)
    state = a.get_state()
    assert len(state) == 10 and isinstance(state, tuple) and state[2:8] == (3, 24, 40, 2, 8, 2)
    assert len(state.message_ta_state) == 1

    np.random.seed(13)  # same clause hypervectors
    b = MultiClassGraphTsetlinMachine(24, 30, (1.5, 2.5), depth=2, message_size=40, message_bits=2, seed=5)
    b.set_state(state)
    assert np.array_equal(b.score(train), a.score(train))
    back = b.get_state()
    assert np.array_equal(back[0], state[0]) and np.array_equal(back[1], state[1])
    assert np.array_equal(back.message_ta_state[0], state.message_ta_state[0])

    # a plain tuple (the reference's) carries no message banks: a fresh model starts them from the initial state
    np.random.seed(13)
    c = MultiClassGraphTsetlinMachine(24, 30, (1.5, 2.5), depth=2, message_size=40, message_bits=2, seed=5)
    c.set_state(tuple(state))
    model = oracle_twin(a, train)
    cfg = model.cfg
    model.ta_state = state[0].reshape(cfg.clauses, cfg.la_chunks, cfg.state_bits).copy()
    model.clause_weights = state[1].reshape(cfg.classes, cfg.clauses).copy()  # message bank: as new_model left it
    assert np.array_equal(c.score(train), o.score(model, train))
    # on an initialised model of the same shape they keep their contents
    a.set_state(tuple(state))
    assert np.array_equal(a.get_state().message_ta_state[0], state.message_ta_state[0])
    # and training goes on from the restored state
    c.step = a.step
    c.set_state(state)
    a.fit(train, Y, epochs=1, incremental=True)
    c.fit(train, Y, epochs=1, incremental=True)
    assert np.array_equal(a.get_state()[0], c.get_state()[0])

    # depth 1: the reference's allocation of depth x the bank; only the first bank is the state
    d1 = MultiClassGraphTsetlinMachine(16, 20, 2.0, seed=3)
    d1.fit(train, Y, epochs=1, incremental=True)
    s1 = d1.get_state()
    e1 = MultiClassGraphTsetlinMachine(16, 20, 2.0, seed=3)
    e1.set_state(tuple(s1))
    assert np.array_equal(e1.score(train), d1.score(train))
    with pytest.raises(Exception, match="sizes"):
        e1.set_state((s1[0][:-1],) + tuple(s1[1:]))


def test_a_later_fit_with_more_labels_than_the_first_is_refused_and_fewer_keep_the_size():
    from graphtsetlinmachine_amd import _abi
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.noisy_xor(200, 50)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=2)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    before = tm.save()
    with pytest.raises(_abi.GtmError, match="sized for 2 outputs"):
        tm.fit(wl.graphs_train, np.where(wl.Y_train == 1, 4, 0), epochs=1, incremental=True)
    after = tm.save()
    assert np.array_equal(before["ta_state"], after["ta_state"]) and tm.number_of_outputs == 2
    # a batch that happens to hold only label 0 trains the same two-output model
    tm.fit(wl.graphs_train, np.zeros_like(wl.Y_train), epochs=1, incremental=True)
    assert tm.number_of_outputs == 2 and tm.score(wl.graphs_test).shape == (50, 2)
    model = oracle_twin(tm, wl.graphs_train)
    cfg = model.cfg
    model.ta_state = before["ta_state"].reshape(cfg.clauses, cfg.la_chunks, cfg.state_bits).copy()
    model.message_ta_state = [b.reshape(cfg.clauses, cfg.message_chunks, cfg.state_bits).copy()
                              for b in before["message_ta_state"]]
    model.clause_weights = before["clause_weights"].reshape(2, -1).copy()
    model.step = 200
    o.fit(model, wl.graphs_train, o.encode_labels(np.zeros_like(wl.Y_train), 2, tm.T))
    assert_same_state(tm, model)
