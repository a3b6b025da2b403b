"""Graphs encoding pinned by closed forms and brute force (no reference import)."""

import hashlib

import numpy as np
import pytest

from graphtsetlinmachine_amd.graphs import Graphs
from tests import helpers


def literal_bits(row, n_literals):
    return [(int(row[k // 32]) >> (k % 32)) & 1 for k in range(n_literals)]


def test_rows_are_or_of_symbol_bits_and_negations():
    np.random.seed(5)
    g = Graphs(2, symbols=["A", "B", "C"], hypervector_size=20, hypervector_bits=3)
    g.set_number_of_graph_nodes(0, 2)
    g.set_number_of_graph_nodes(1, 1)
    g.prepare_node_configuration()
    for gid, name in [(0, "x"), (0, "y"), (1, "z")]:
        g.add_graph_node(gid, name, 0)
    g.prepare_edge_configuration()
    g.add_graph_node_property(0, "x", "A")
    g.add_graph_node_property(0, "x", "C")
    g.add_graph_node_property(1, "z", "B")
    g.encode()
    hv = g.hypervector_size
    assert g.X.shape == (3, 2) and g.X.dtype == np.uint32
    expected_sets = [set(g.hypervectors[0]) | set(g.hypervectors[2]), set(), set(g.hypervectors[1])]
    for row, on in zip(g.X, expected_sets):
        bits = literal_bits(row, 64)
        for k in range(hv):
            assert bits[k] == (1 if k in on else 0)
            assert bits[k + hv] == 1 - bits[k]  # negated literal
        assert sum(bits[2 * hv:]) == 0  # padding stays clear
        assert sum(bits) == hv
    assert list(g.node_index) == [0, 2]
    assert g.max_number_of_graph_nodes == 2 and g.max_number_of_graph_node_chunks == 1


def test_hypervectors_follow_the_global_numpy_stream():
    np.random.seed(11)
    g = Graphs(1, symbols=list("abcde"), hypervector_size=32, hypervector_bits=2)
    np.random.seed(11)
    want = np.stack([np.random.choice(np.arange(32), size=2, replace=False) for _ in range(5)])
    assert np.array_equal(g.hypervectors, want.astype(np.uint32))
    assert all(len(set(r)) == 2 for r in g.hypervectors)


def test_double_hashing_and_one_hot_tables():
    g = Graphs(1, symbols=list(range(300)), hypervector_size=128, double_hashing=True)
    i = np.arange(300)
    assert np.array_equal(g.hypervectors[:, 0], i % 128)
    assert np.array_equal(g.hypervectors[:, 1], 127 - (i % 127))  # prevprime(128) == 127
    assert g.hypervector_bits == 2
    h = Graphs(1, symbols=list("abc"), hypervector_size=999, one_hot_encoding=True)
    assert h.hypervector_size == 3 and h.hypervector_bits == 1
    assert np.array_equal(h.hypervectors[:, 0], [0, 1, 2])
    assert h.number_of_hypervector_chunks == 1


def tutorial_graphs(n, xs):
    """The Noisy XOR construction of the reference's tutorial (README.md:70-146)."""
    np.random.seed(3)
    g = Graphs(n, symbols=["A", "B"], hypervector_size=32, hypervector_bits=2)
    for i in range(n):
        g.set_number_of_graph_nodes(i, 2)
    g.prepare_node_configuration()
    for i in range(n):
        g.add_graph_node(i, "Node 1", 1)
        g.add_graph_node(i, "Node 2", 1)
    g.prepare_edge_configuration()
    for i in range(n):
        g.add_graph_node_edge(i, "Node 1", "Node 2", "Plain")
        g.add_graph_node_edge(i, "Node 2", "Node 1", "Plain")
    for i in range(n):
        g.add_graph_node_property(i, "Node 1", xs[i][0])
        g.add_graph_node_property(i, "Node 2", xs[i][1])
    g.encode()
    return g


def test_tutorial_graph_layout():
    xs = [("A", "B"), ("B", "B"), ("A", "A")]
    g = tutorial_graphs(3, xs)
    assert g.X.shape == (6, 2)
    assert np.array_equal(g.edge, [[1, 0], [0, 0]] * 3)
    assert np.array_equal(g.edge_index, np.arange(6))
    assert np.array_equal(g.node_index, [0, 2, 4])
    assert np.array_equal(g.number_of_graph_node_edges, np.ones(6))
    assert g.edge_type_id == {"Plain": 0} and g.node_type_id == {"Plain": 0}
    assert np.array_equal(g.X[0], g.X[4]) and np.array_equal(g.X[1], g.X[2])
    m = hashlib.sha256()
    m.update(g.X.tobytes())
    m.update(g.edge.tobytes())
    assert g.signature == m.digest()
    assert len(g) == 3


@pytest.mark.parametrize("encoder", ["native", "numpy"])
def test_bulk_builders_equal_single_calls(encoder, monkeypatch):
    from graphtsetlinmachine_amd import graphs as graphs_module

    if encoder == "numpy":
        monkeypatch.setenv("GTM_NO_NATIVE_ENCODER", "1")
        assert graphs_module._native_encoder() is None
    else:
        assert graphs_module._native_encoder() is not None, "libgtm_encode.so has not been built"
    rng = np.random.default_rng(0)
    n, nodes = 7, 5
    np.random.seed(9)
    a = Graphs(n, symbols=list(range(6)), hypervector_size=24, hypervector_bits=2)
    np.random.seed(9)
    b = Graphs(n, symbols=list(range(6)), hypervector_size=24, hypervector_bits=2)
    for g in (a, b):
        g.number_of_graph_nodes[:] = nodes
        g.prepare_node_configuration()
    degree = rng.integers(0, 3, size=(n, nodes))
    types = rng.choice(["p", "q"], size=(n, nodes))
    for i in range(n):
        for j in range(nodes):
            a.add_graph_node(i, j, int(degree[i, j]), str(types[i, j]))
    b.add_graph_nodes(degree.reshape(-1), node_types=types.reshape(-1))
    a.prepare_edge_configuration()
    b.prepare_edge_configuration()
    gid, src, dst, kinds = [], [], [], []
    for i in range(n):
        for j in range(nodes):
            for _ in range(degree[i, j]):
                d, k = int(rng.integers(nodes)), str(rng.choice(["L", "R", "U"]))
                a.add_graph_node_edge(i, j, d, k)
                gid.append(i), src.append(j), dst.append(d), kinds.append(k)
    b.add_graph_node_edges(gid, src, dst, kinds)
    rows, syms = [], []
    for i in range(n):
        for j in range(nodes):
            for s in rng.choice(6, size=rng.integers(0, 4), replace=False):
                a.add_graph_node_property(i, j, int(s))
                rows.append(i * nodes + j), syms.append(int(s))
    half = len(rows) // 2
    b.add_graph_node_properties(rows[:half], syms[:half])
    member = np.zeros((n * nodes, 6), dtype=bool)
    member[rows[half:], syms[half:]] = True
    b.add_graph_node_property_matrix(0, member)
    a.encode()
    b.encode()
    for name in ("X", "edge", "node_type", "number_of_graph_node_edges", "node_index", "edge_index"):
        assert np.array_equal(getattr(a, name), getattr(b, name)), name
    assert a.signature == b.signature
    assert a.node_type_id == b.node_type_id and a.edge_type_id == b.edge_type_id


def test_prefix_sums_and_ragged_sizes():
    g = helpers.random_graphs(21, n_graphs=9, max_nodes=50)
    counts = g.number_of_graph_nodes.astype(np.int64)
    assert np.array_equal(g.node_index, np.cumsum(counts) - counts)
    e = g.number_of_graph_node_edges.astype(np.int64)
    assert np.array_equal(g.edge_index, np.cumsum(e) - e)
    assert g.edge.shape == (e.sum(), 2)
    owner = np.repeat(np.arange(9), counts)
    per_edge_owner = np.repeat(owner, e)
    assert (g.edge[:, 0] < counts[per_edge_owner]).all()  # destinations are graph-local
    pc = np.unpackbits(g.X.view(np.uint8), axis=1).sum(axis=1)
    assert (pc == g.hypervector_size).all()


def test_misuse_exits_like_the_reference():
    g = Graphs(1, symbols=["A"], hypervector_size=8, hypervector_bits=1)
    g.set_number_of_graph_nodes(0, 2)
    g.prepare_node_configuration()
    g.add_graph_node(0, "a", 1)
    g.add_graph_node(0, "b", 1)
    g.prepare_edge_configuration()
    g.add_graph_node_edge(0, "a", "b", "t")
    with pytest.raises(SystemExit) as too_many:
        g.add_graph_node_edge(0, "a", "b", "t")
    assert too_many.value.code == -1
    with pytest.raises(SystemExit) as missing:
        g.encode()  # node b still misses its edge
    assert missing.value.code == -1 and "misses edges" in str(missing.value)


def test_subsetting_matches_direct_construction_and_shares_vocabulary():
    g = helpers.random_graphs(33, n_graphs=8, max_nodes=12, edge_types=("x", "y"))
    sub = g[[5, 0, 5]]
    assert len(sub) == 3 and sub.symbol_id is g.symbol_id and sub.hypervectors is g.hypervectors
    for new, old in enumerate([5, 0, 5]):
        n = int(g.number_of_graph_nodes[old])
        a, b = int(sub.node_index[new]), int(g.node_index[old])
        assert np.array_equal(sub.X[a:a + n], g.X[b:b + n])
        assert np.array_equal(sub.node_type[a:a + n], g.node_type[b:b + n])
        ne = int(g.number_of_graph_node_edges[b:b + n].sum())
        ea, eb = (int(sub.edge_index[a]), int(g.edge_index[b])) if n else (0, 0)
        assert np.array_equal(sub.edge[ea:ea + ne], g.edge[eb:eb + ne])
    assert len(g[2:4]) == 2 and len(g[-1]) == 1
    with pytest.raises(IndexError):
        g[8]
    with pytest.raises(ValueError):
        g[[]]
    child = Graphs(1, init_with=g)
    child.set_number_of_graph_nodes(0, 1)
    child.prepare_node_configuration()
    child.add_graph_node(0, "n", 0, "brand-new-type")
    assert "brand-new-type" in g.node_type_id  # shared dict, as in the reference


def test_print_graph_writes_the_reference_format(capsys):
    """graphs.py:164-206: one line of nodes with the symbols each holds ('*' for the others), one
    line per edge with its global slot, a blank line after each node's edges."""
    from graphtsetlinmachine_amd.graphs import Graphs

    g = Graphs(1, symbols=["A", "B"], hypervector_size=8, hypervector_bits=1, one_hot_encoding=True)
    g.set_number_of_graph_nodes(0, 2)
    g.prepare_node_configuration()
    g.add_graph_node(0, "n0", 1)
    g.add_graph_node(0, "n1", 1)
    g.prepare_edge_configuration()
    g.add_graph_node_edge(0, "n0", "n1", "Plain")
    g.add_graph_node_edge(0, "n1", "n0", "Other")
    g.add_graph_node_property(0, "n0", "A")
    g.add_graph_node_property(0, "n1", "B")
    g.encode()
    g.print_graph(0)
    out = capsys.readouterr().out
    assert out == ("Printing nodes of Graph#0:\nNode#0( A * ) Node#1( * B ) \n\n"
                   "Printing edges of Graph#0:\nEdge#0 SrcNode#0 DestNode#1 EdgeType#0\n\n"
                   "Edge#1 SrcNode#1 DestNode#0 EdgeType#1\n\n\n\n")


@pytest.mark.parametrize("hv_size, hv_bits", [(20, 3), (64, 2), (1024, 2), (37, 1)])
def test_the_native_encoder_and_the_numpy_forms_build_the_same_rows(hv_size, hv_bits, monkeypatch):
    """csrc/encode.c (the reference's per-property loop, graphs.py:148-162, over whole arrays) against
    the vectorised NumPy forms: repeated pairs, rows that already hold properties, both entry points."""
    from graphtsetlinmachine_amd import graphs as graphs_module

    assert graphs_module._native_encoder() is not None, "libgtm_encode.so has not been built"
    rng = np.random.default_rng(hv_size)
    n_symbols, n_graphs, nodes = 23, 40, 50

    def build():
        np.random.seed(hv_size)
        g = Graphs(n_graphs, symbols=list(range(n_symbols)), hypervector_size=hv_size, hypervector_bits=hv_bits)
        g.number_of_graph_nodes[:] = nodes
        g.prepare_node_configuration()
        g.add_graph_nodes(0)
        g.prepare_edge_configuration()
        return g

    rows = rng.integers(0, n_graphs * nodes, size=6000)
    syms = rng.integers(0, n_symbols, size=6000)
    member = rng.random((700, n_symbols)) < 0.2
    native, plain = build(), build()
    native.add_graph_node_properties(rows, syms)
    native.add_graph_node_property_matrix(300, member)
    native.add_graph_node_property_matrix(900, member.astype(np.uint8) * 7)  # any non-zero value counts
    monkeypatch.setenv("GTM_NO_NATIVE_ENCODER", "1")
    plain.add_graph_node_properties(rows, syms)
    plain.add_graph_node_property_matrix(300, member)
    plain.add_graph_node_property_matrix(900, member.astype(np.uint8) * 7)
    assert np.array_equal(native.X, plain.X)
    # and both equal the single calls on a few rows
    single = build()
    for r, s_ in zip(rows[:300].tolist(), syms[:300].tolist()):
        single.add_graph_node_property(r // nodes, r % nodes, s_)
    check = build()
    monkeypatch.delenv("GTM_NO_NATIVE_ENCODER")
    check.add_graph_node_properties(rows[:300], syms[:300])
    assert np.array_equal(check.X, single.X)
    with pytest.raises(IndexError):
        check.add_graph_node_properties([n_graphs * nodes], [0])
    with pytest.raises(IndexError):
        check.add_graph_node_properties([0], [n_symbols])
    with pytest.raises(IndexError):
        check.add_graph_node_property_matrix(n_graphs * nodes - 10, member)
