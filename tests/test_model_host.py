"""Host-side logic of the model classes that needs no GPU: the state file
formats, the guard on the number of outputs, and the clause hypervector tables
(tm.py:90-106, 415-418)."""

import numpy as np
import pytest

from graphtsetlinmachine_amd import _abi
from graphtsetlinmachine_amd import tm as tm_module
from graphtsetlinmachine_amd.graphs import Graphs
from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine, MultiOutputGraphTsetlinMachine

# the keys of the reference's save() dict, tm.py:328-354
REFERENCE_KEYS = [
    "ta_state", "message_ta_state", "clause_weights", "hypervectors", "number_of_outputs", "number_of_literals",
    "number_of_message_literals", "min_y", "max_y", "negative_clauses", "max_number_of_graph_nodes",
    "number_of_clauses", "T", "s", "q", "max_included_literals", "boost_true_positive_feedback",
    "number_of_state_bits", "depth", "message_size", "message_bits", "double_hashing", "one_hot_encoding",
]


def reference_shaped_state(rng, clauses=6, literals=40, depth=3, state_bits=8, outputs=3, message_size=24):
    la, mc = (literals - 1) // 32 + 1, (2 * message_size - 1) // 32 + 1
    return {
        "ta_state": rng.integers(0, 2**32, size=clauses * la * state_bits, dtype=np.uint64).astype(np.uint32),
        "message_ta_state": [rng.integers(0, 2**32, size=clauses * mc * state_bits, dtype=np.uint64).astype(np.uint32)
                             for _ in range(depth - 1)],
        "clause_weights": rng.integers(-9, 10, size=outputs * clauses).astype(np.int32),
        "hypervectors": rng.integers(0, message_size, size=(clauses, 2)).astype(np.uint32),
        "number_of_outputs": outputs, "number_of_literals": literals,
        "number_of_message_literals": 2 * message_size, "min_y": None, "max_y": None, "negative_clauses": 1,
        "max_number_of_graph_nodes": 17, "number_of_clauses": clauses, "T": 25, "s": (1.5, 2.0, 3.25), "q": 1.0,
        "max_included_literals": 11, "boost_true_positive_feedback": 1, "number_of_state_bits": state_bits,
        "depth": depth, "message_size": message_size, "message_bits": 2, "double_hashing": False,
        "one_hot_encoding": False,
    }


def test_npz_state_file_round_trips_without_pickle(tmp_path):
    state = reference_shaped_state(np.random.default_rng(1))
    assert list(state) == REFERENCE_KEYS
    path = str(tmp_path / "model.npz")
    tm_module.write_state_npz(state, path)
    with np.load(path, allow_pickle=False) as z:  # nothing in the archive needs unpickling
        assert z["ta_state"].dtype == np.uint32 and z["clause_weights"].dtype == np.int32
        assert "min_y" not in z.files  # None is stored as absence
    back = tm_module.read_state_npz(path)
    assert set(REFERENCE_KEYS) <= set(back)
    for key in REFERENCE_KEYS:
        if key == "message_ta_state":
            assert len(back[key]) == 2 and all(np.array_equal(a, b) for a, b in zip(back[key], state[key]))
        elif isinstance(state[key], np.ndarray):
            assert back[key].dtype == state[key].dtype and np.array_equal(back[key], state[key])
        else:
            assert back[key] == state[key] and type(back[key]) is type(state[key]), key
    # the generator position travels when present, with all 64 bits of the seed
    state["rng_seed"], state["rng_step"] = 2**64 - 3, 123456789012
    tm_module.write_state_npz(state, path)
    back = tm_module.read_state_npz(path)
    assert back["rng_seed"] == 2**64 - 3 and back["rng_step"] == 123456789012


def test_a_pickled_state_is_read_without_running_what_it_names(tmp_path):
    """A pickle can name any importable callable and have it called while it loads.  The reader of
    state files rebuilds arrays, scalars and plain containers only: the reference's dict comes back
    equal, and a file that names anything else is refused before that thing runs."""
    import pickle

    state = reference_shaped_state(np.random.default_rng(2))
    state["q"] = np.float64(1.0)  # NumPy scalars travel too (numpy.core.multiarray.scalar)
    path = str(tmp_path / "model.pkl")
    with open(path, "wb") as f:
        pickle.dump(state, f)
    back = tm_module.read_state_pickle(path)
    assert list(back) == REFERENCE_KEYS
    for key in REFERENCE_KEYS:
        if key == "message_ta_state":
            assert all(np.array_equal(a, b) for a, b in zip(back[key], state[key]))
        elif isinstance(state[key], np.ndarray):
            assert back[key].dtype == state[key].dtype and np.array_equal(back[key], state[key])
        else:
            assert back[key] == state[key]

    marker = tmp_path / "ran"

    class Payload:
        def __reduce__(self):
            import os

            return (os.system, ("touch %s" % marker,))

    for poisoned in (Payload(), dict(state, T=Payload()), {"ta_state": [Payload()]}):
        with open(path, "wb") as f:
            pickle.dump(poisoned, f)
        with pytest.raises(pickle.UnpicklingError, match="only NumPy arrays"):
            tm_module.read_state_pickle(path)
        assert not marker.exists()
    # the model's load() goes through the same reader (no device is touched before the file is read)
    with pytest.raises(pickle.UnpicklingError, match="only NumPy arrays"):
        MultiClassGraphTsetlinMachine(10, 20, 1.0).load(fname=path)
    assert not marker.exists()
    # something that is not the dict of save()
    with open(path, "wb") as f:
        pickle.dump([1, 2, 3], f)
    with pytest.raises(pickle.UnpicklingError, match="not the dict"):
        tm_module.read_state_pickle(path)


def test_more_outputs_than_allocated_is_refused_before_any_device_call(monkeypatch):
    """The weight buffer and the tile geometry are sized at the first fit; a later batch with a
    higher label must not reach the kernels (an out-of-bounds device write)."""
    called = []
    monkeypatch.setattr(_abi, "call", lambda *a, **k: called.append(a))
    monkeypatch.setattr(tm_module, "_device", lambda: called.append("device"))
    tm = MultiClassGraphTsetlinMachine(10, 20, 1.0)
    tm.initialized = True
    tm._allocated_outputs = 3
    tm.number_of_outputs = 3
    with pytest.raises(_abi.GtmError, match="sized for 3 outputs"):
        tm.fit(None, np.array([0, 1, 5]), epochs=1, incremental=True)
    assert called == []
    # fewer labels in a batch keep the model's size
    assert tm._outputs_for(2) == 3
    # a config for another number of outputs than the buffers hold is never built
    tm.number_of_outputs = 4
    with pytest.raises(_abi.GtmError, match="allocated for"):
        tm._config(5)
    mo = MultiOutputGraphTsetlinMachine(10, 20, 1.0)
    mo.initialized = True
    mo._allocated_outputs = 3
    mo.number_of_outputs = 3
    with pytest.raises(_abi.GtmError):
        mo.fit(None, np.zeros((4, 2), dtype=np.int64), epochs=1, incremental=True)
    with pytest.raises(_abi.GtmError):
        mo.fit(None, np.zeros((4, 5), dtype=np.int64), epochs=1, incremental=True)
    assert called == []


def test_clause_hypervector_tables_follow_the_reference_formulas():
    """tm.py:90-106: double hashing gives clause i the bits (i mod M, p - (i mod p)), p the largest
    prime below M; one-hot gives one bit per clause, placed when the edge types are known
    (tm.py:415-418): M = clauses * max(1, edge types), h[i] = i * edge types."""
    from sympy import prevprime

    tm = MultiClassGraphTsetlinMachine(50, 20, 1.0, depth=2, message_size=32, message_bits=5, double_hashing=True)
    p = int(prevprime(32))
    assert p == 31 and tm.message_bits == 2 and tm.hypervectors.dtype == np.uint32
    for i in (0, 1, 30, 31, 32, 49):
        assert tuple(tm.hypervectors[i]) == (i % 32, p - (i % p))
    assert tm.hypervectors.max() < 32

    one = MultiClassGraphTsetlinMachine(7, 20, 1.0, depth=2, message_size=999, message_bits=4, one_hot_encoding=True)
    assert one.message_bits == 1 and one.hypervectors.shape == (7, 1)

    class G:  # the attributes _init reads
        edge_type_id = {"a": 0, "b": 1, "c": 2}
        hypervector_size = 16
        max_number_of_graph_nodes = 4

    one.number_of_outputs = 2
    one._allocate = lambda: None
    one._init(G)
    assert one.message_size == 21 and list(one.hypervectors[:, 0]) == [0, 3, 6, 9, 12, 15, 18]
    assert one.number_of_message_literals == 42 and one.number_of_message_chunks == 2
    # rotating by an edge type keeps the clauses' bits apart: (h + t) mod M is unique per (clause, type)
    seen = {(int(h) + t) % 21 for h in one.hypervectors[:, 0] for t in range(3)}
    assert len(seen) == 21

    G.edge_type_id = {}
    none = MultiClassGraphTsetlinMachine(5, 20, 1.0, depth=2, one_hot_encoding=True)
    none.number_of_outputs = 2
    none._allocate = lambda: None
    none._init(G)
    assert none.message_size == 5 and not none.hypervectors.any()


def test_a_foreign_node_name_after_the_bulk_builder_is_appended_like_the_reference_dict():
    g = Graphs(2, symbols=["a"], hypervector_size=8, hypervector_bits=1)
    g.set_number_of_graph_nodes(0, 3)
    g.set_number_of_graph_nodes(1, 2)
    g.prepare_node_configuration()
    g.add_graph_nodes(0)
    g.add_graph_node(0, 1, 0, "Other")  # a known name: same row, new type
    assert g.node_type[1] == g.node_type_id["Other"]
    # graph 1 has rows for two nodes; a third, foreign name gets the next id as a dict would give it
    # (the reference writes past the graph's rows in that case too; here it is the last graph, so guard the row)
    names_before = g.graph_node_id[0]
    assert 2 in names_before and "x" not in names_before
    assert type(names_before).__name__ == "_RangeNames"
    g.add_graph_node(0, "x", 0)  # id 3 = first row of graph 1
    assert isinstance(g.graph_node_id[0], dict) and g.graph_node_id[0]["x"] == 3 and g.graph_node_id[0][2] == 2


def test_subsetting_copies_only_the_edges_added_so_far():
    """graphs.py:288-296 copies graph_node_edge_counter edges per node; an incomplete data set then
    fails its subset's encode() as the reference's does, without reading unset edge rows."""
    from graphtsetlinmachine_amd.graphs import GraphsError

    g = Graphs(2, symbols=["a"], hypervector_size=8, hypervector_bits=1)
    for i in range(2):
        g.set_number_of_graph_nodes(i, 2)
    g.prepare_node_configuration()
    for i in range(2):
        g.add_graph_node(i, "p", 2)
        g.add_graph_node(i, "q", 1)
    g.prepare_edge_configuration()
    g.edge[:] = 0xDEAD
    g.add_graph_node_edge(1, "p", "q", "t")
    g.add_graph_node_edge(1, "q", "p", "t")
    with pytest.raises(GraphsError):
        g[[1]]
    g.add_graph_node_edge(1, "p", "p", "u")
    for _ in range(2):
        g.add_graph_node_edge(0, "p", "q", "t")
    g.add_graph_node_edge(0, "q", "q", "u")
    g.encode()
    sub = g[[1]]
    assert sub.edge.tolist() == [[1, 0], [0, 1], [0, 0]]
