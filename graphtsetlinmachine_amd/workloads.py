"""Seeded synthetic workloads: the five benchmark configurations and the README's sequence task.

Each builder returns a ``Workload`` with encoded train/test ``Graphs``, labels
and the constructor arguments of ``MultiClassGraphTsetlinMachine`` for that
configuration.  Graph counts can be scaled down (tests use a few dozen graphs,
the benchmark uses thousands); shapes per graph never change.

The graph shapes follow the reference's demos: two-node XOR graphs with one
'Plain' edge each way (examples/NoisyXORDemo.py:49-64), one node per image with
"x:y" pixel symbols (examples/MNISTVanillaDemo.py:46-48,74-75), patch nodes with
pixel-offset symbols plus thermometer-coded position
(examples/CIFAR10Demo.py:65-74,100-113), chains with 'Left'/'Right' edges
(examples/SequenceClassificationDemo.py:54-72).
"""

from dataclasses import dataclass

import numpy as np
from numpy.lib.stride_tricks import sliding_window_view

from .graphs import Graphs


@dataclass
class Workload:
    name: str
    graphs_train: Graphs
    Y_train: np.ndarray
    graphs_test: Graphs
    Y_test: np.ndarray
    params: dict  # kwargs of MultiClassGraphTsetlinMachine
    classes: int


def _seeded_graphs(seed, *args, **kwargs):
    """Graphs() draws symbol hypervectors from NumPy's global generator; seed
    it for the draw and put the caller's state back afterwards."""
    saved = np.random.get_state()
    np.random.seed(seed)
    try:
        return Graphs(*args, **kwargs)
    finally:
        np.random.set_state(saved)


def _uniform_nodes(graphs, nodes_per_graph):
    graphs.number_of_graph_nodes[:] = nodes_per_graph
    graphs.prepare_node_configuration()


# ------------------------------------------------------------------ config 1


def noisy_xor(n_train=10000, n_test=10000, seed=1235, noise=0.01):
    rng = np.random.default_rng(seed)

    def build(n, parent, flip):
        if parent is None:
            g = _seeded_graphs(seed, n, symbols=["A", "B"], hypervector_size=32, hypervector_bits=2)
        else:
            g = Graphs(n, init_with=parent)
        _uniform_nodes(g, 2)
        g.add_graph_nodes(1)
        g.prepare_edge_configuration()
        ids = np.arange(n)
        g.add_graph_node_edges(np.r_[ids, ids], np.r_[np.zeros(n, int), np.ones(n, int)],
                               np.r_[np.ones(n, int), np.zeros(n, int)], "Plain")
        x = rng.integers(0, 2, size=(n, 2))
        g.add_graph_node_properties(np.arange(2 * n), x.reshape(-1))
        y = (x[:, 0] != x[:, 1]).astype(np.uint32)
        if flip:
            y = np.where(rng.random(n) <= noise, 1 - y, y).astype(np.uint32)
        g.encode()
        return g, y

    gtr, ytr = build(n_train, None, True)
    gte, yte = build(n_test, gtr, False)
    params = dict(number_of_clauses=10, T=100, s=1.0, depth=2, message_size=256, message_bits=2)
    return Workload("noisy_xor", gtr, ytr, gte, yte, params, 2)


# ------------------------------------------------------- configs 2 and 3 data


def _binary_images(rng, templates, n):
    """Class-conditional Bernoulli pixels plus 5 % flips."""
    y = rng.integers(0, templates.shape[0], size=n).astype(np.uint32)
    img = rng.random((n, 28, 28)) < templates[y]
    img ^= rng.random((n, 28, 28)) < 0.05
    return img, y


def _templates(rng):
    return np.where(rng.random((10, 28, 28)) < 0.5, 0.8, 0.1)


def single_node_images(n_train=60000, n_test=10000, seed=1236):
    rng = np.random.default_rng(seed)
    templates = _templates(rng)
    symbols = ["%d:%d" % (x, y) for x in range(28) for y in range(28)]

    def build(n, parent):
        img, y = _binary_images(rng, templates, n)
        if parent is None:
            g = _seeded_graphs(seed, n, symbols=symbols, hypervector_size=2048, hypervector_bits=2)
        else:
            g = Graphs(n, init_with=parent)
        _uniform_nodes(g, 1)
        g.add_graph_nodes(0)
        g.prepare_edge_configuration()
        g.add_graph_node_property_matrix(0, img.reshape(n, 784))
        g.encode()
        return g, y

    gtr, ytr = build(n_train, None)
    gte, yte = build(n_test, gtr)
    params = dict(number_of_clauses=2500, T=3125, s=10.0, depth=1)
    return Workload("single_node_images", gtr, ytr, gte, yte, params, 10)


def convolutional_images(n_train=60000, n_test=10000, seed=1237, patch=10):
    """19x19 = 361 patch nodes per image, no edges, 138 symbols."""
    rng = np.random.default_rng(seed)
    templates = _templates(rng)
    dim = 28 - patch + 1
    symbols = []
    for i in range(dim):
        symbols.append("C:%d" % i)
        symbols.append("R:%d" % i)
    symbols += list(range(patch * patch))
    pos = np.arange(dim)
    thermo = (pos[None, :] <= pos[:, None])  # thermo[q][i] = symbol i present at coordinate q

    def build(n, parent):
        img, y = _binary_images(rng, templates, n)
        if parent is None:
            g = _seeded_graphs(seed, n, symbols=symbols, hypervector_size=128, hypervector_bits=2)
        else:
            g = Graphs(n, init_with=parent)
        _uniform_nodes(g, dim * dim)
        g.add_graph_nodes(0)
        g.prepare_edge_configuration()
        block = 512
        for a in range(0, n, block):
            b = min(n, a + block)
            windows = sliding_window_view(img[a:b], (patch, patch), axis=(1, 2))  # [b][q][r][p][p]
            member = np.zeros((b - a, dim, dim, len(symbols)), dtype=np.uint8)
            member[:, :, :, 0 : 2 * dim : 2] = thermo[None, :, None, :]  # C:0..q
            member[:, :, :, 1 : 2 * dim : 2] = thermo[None, None, :, :]  # R:0..r
            member[:, :, :, 2 * dim :] = windows.reshape(b - a, dim, dim, patch * patch)
            g.add_graph_node_property_matrix(a * dim * dim, member.reshape(-1, len(symbols)))
        g.encode()
        return g, y

    gtr, ytr = build(n_train, None)
    gte, yte = build(n_test, gtr)
    params = dict(number_of_clauses=2500, T=3125, s=10.0, depth=1)
    return Workload("convolutional_images", gtr, ytr, gte, yte, params, 10)


# ------------------------------------------------------------------ config 4


def sequence_chains(n_train=20000, n_test=5000, seed=1238, length=1000):
    """Chains of `length` tokens; class 1 iff some 'A' is followed within 3
    positions by 'B' (planted in half of the sequences, scrubbed from the rest)."""
    rng = np.random.default_rng(seed)
    alphabet = [chr(ord("A") + i) for i in range(26)]

    def sequences(n):
        seq = rng.integers(0, 26, size=(n, length))
        # scrub accidental patterns: a 'B' up to 3 places after an 'A' becomes C..Z
        is_a = seq == 0
        near_a = np.zeros_like(is_a)
        for d in (1, 2, 3):
            near_a[:, d:] |= is_a[:, :-d]
        bad = near_a & (seq == 1)
        seq[bad] = rng.integers(2, 26, size=int(bad.sum()))
        y = (rng.random(n) < 0.5).astype(np.uint32)
        planted = np.flatnonzero(y)
        p = rng.integers(0, length - 3, size=planted.size)
        d = rng.integers(1, 4, size=planted.size)
        seq[planted, p] = 0
        seq[planted, p + d] = 1
        return seq, y

    def build(n, parent):
        seq, y = sequences(n)
        if parent is None:
            g = _seeded_graphs(seed, n, symbols=alphabet, hypervector_size=64, hypervector_bits=2)
        else:
            g = Graphs(n, init_with=parent)
        _uniform_nodes(g, length)
        degree = np.full((n, length), 2, dtype=np.uint32)
        degree[:, 0] = 1
        degree[:, -1] = 1
        if length == 1:
            degree[:] = 0
        g.add_graph_nodes(degree.reshape(-1))
        g.prepare_edge_configuration()
        gid = np.repeat(np.arange(n), length - 1)
        left_src = np.tile(np.arange(1, length), n)
        right_src = np.tile(np.arange(0, length - 1), n)
        # per node the reference adds 'Left' before 'Right'
        # (examples/SequenceClassificationDemo.py:64-72)
        g.add_graph_node_edges(gid, left_src, left_src - 1, "Left")
        g.add_graph_node_edges(gid, right_src, right_src + 1, "Right")
        g.add_graph_node_properties(np.arange(n * length), seq.reshape(-1))
        g.encode()
        return g, y

    gtr, ytr = build(n_train, None)
    gte, yte = build(n_test, gtr)
    params = dict(number_of_clauses=200, T=400, s=1.0, depth=2, message_size=512, message_bits=2)
    return Workload("sequence_chains", gtr, ytr, gte, yte, params, 2)


# ------------------------------------------------------------------ config 5


def colour_convolution(n_train=50000, n_test=10000, seed=1239, patch=4, levels=8):
    """32x32x3 Gaussian-blob images, 8-level thermometer code per channel,
    4x4 patches -> 29x29 = 841 nodes on a 4-neighbour grid with one edge type
    per direction."""
    rng = np.random.default_rng(seed)
    size = 32
    dim = size - patch + 1
    yy, xx = np.mgrid[0:size, 0:size]
    templates = np.zeros((10, size, size, 3))
    for k in range(10):
        for c in range(3):
            for _ in range(3):
                cx, cy = rng.uniform(4, size - 4, size=2)
                sigma = rng.uniform(2.5, 6.0)
                templates[k, :, :, c] += rng.uniform(0.4, 1.0) * np.exp(
                    -((xx - cx) ** 2 + (yy - cy) ** 2) / (2 * sigma * sigma))
    templates = np.clip(templates, 0.0, 1.0)
    symbols = []
    for i in range(dim):
        symbols.append("C:%d" % i)
        symbols.append("R:%d" % i)
    symbols += list(range(patch * patch * 3 * levels))
    pos = np.arange(dim)
    thermo = (pos[None, :] <= pos[:, None])
    cuts = (np.arange(levels) + 1.0) / (levels + 1.0)

    # grid edges in a fixed per-node order: Up, Down, Left, Right
    q, r = np.mgrid[0:dim, 0:dim]
    node = (q * dim + r).reshape(-1)
    qf, rf = q.reshape(-1), r.reshape(-1)
    src, dst, kind = [], [], []
    for name, ok, delta in (("Up", qf > 0, -dim), ("Down", qf < dim - 1, dim),
                            ("Left", rf > 0, -1), ("Right", rf < dim - 1, 1)):
        src.append(node[ok])
        dst.append(node[ok] + delta)
        kind.append(name)
    degree = (qf > 0).astype(int) + (qf < dim - 1) + (rf > 0) + (rf < dim - 1)

    def build(n, parent):
        y = rng.integers(0, 10, size=n).astype(np.uint32)
        if parent is None:
            g = _seeded_graphs(seed, n, symbols=symbols, hypervector_size=1024, hypervector_bits=2)
        else:
            g = Graphs(n, init_with=parent)
        _uniform_nodes(g, dim * dim)
        g.add_graph_nodes(np.tile(degree, n))
        g.prepare_edge_configuration()
        for s_, d_, k_ in zip(src, dst, kind):
            g.add_graph_node_edges(np.repeat(np.arange(n), s_.size), np.tile(s_, n), np.tile(d_, n), k_)
        block = 32
        for a in range(0, n, block):
            b = min(n, a + block)
            img = templates[y[a:b]] + rng.normal(0.0, 0.1, size=(b - a, size, size, 3))
            coded = img[..., None] > cuts  # [b][32][32][3][levels]
            coded = coded.reshape(b - a, size, size, 3 * levels)
            windows = sliding_window_view(coded, (patch, patch), axis=(1, 2))  # [b][q][r][3L][p][p]
            member = np.zeros((b - a, dim, dim, len(symbols)), dtype=np.uint8)
            member[:, :, :, 0 : 2 * dim : 2] = thermo[None, :, None, :]
            member[:, :, :, 1 : 2 * dim : 2] = thermo[None, None, :, :]
            member[:, :, :, 2 * dim :] = windows.reshape(b - a, dim, dim, -1)
            g.add_graph_node_property_matrix(a * dim * dim, member.reshape(-1, len(symbols)))
        g.encode()
        return g, y

    gtr, ytr = build(n_train, None)
    gte, yte = build(n_test, gtr)
    params = dict(number_of_clauses=8000, T=10000, s=15.0, depth=3, message_size=1024, message_bits=2)
    return Workload("colour_convolution", gtr, ytr, gte, yte, params, 10)


# ----------------------------------------------- the README's sequence task


def runs_of_a(n_train=40000, n_test=40000, seed=1240, classes=3, max_length=10, noise=0.01):
    """The task of the reference's sequence demo (README.md:194-208,
    examples/SequenceClassificationDemo.py:48-84): chains of 3..max_length nodes
    with 'Left'/'Right' edges, one run of y + 1 consecutive 'A's somewhere, the
    class is y.  A node sees only its own symbol, so the classes can only be told
    apart through the messages: learning it needs every part of a model with
    message layers to work."""
    rng = np.random.default_rng(seed)

    def build(n, parent, flip):
        if parent is None:
            g = _seeded_graphs(seed, n, symbols=["A"], hypervector_size=256, hypervector_bits=2)
        else:
            g = Graphs(n, init_with=parent)
        lengths = rng.integers(classes, max_length + 1, size=n)
        g.number_of_graph_nodes[:] = lengths
        g.prepare_node_configuration()
        local = np.concatenate([np.arange(m) for m in lengths])
        gid = np.repeat(np.arange(n), lengths)
        last = np.repeat(lengths, lengths) - 1
        degree = np.where((local > 0) & (local < last), 2, 1).astype(np.uint32)
        g.add_graph_nodes(degree)
        g.prepare_edge_configuration()
        # per node the reference adds 'Left' before 'Right' (examples/SequenceClassificationDemo.py:64-72)
        has_left, has_right = local > 0, local < last
        g.add_graph_node_edges(gid[has_left], local[has_left], local[has_left] - 1, "Left")
        g.add_graph_node_edges(gid[has_right], local[has_right], local[has_right] + 1, "Right")
        y = rng.integers(0, classes, size=n).astype(np.uint32)
        end = rng.integers(y, lengths)  # the run ends at node `end`, inclusive
        rows = np.concatenate([g.node_index[i] + np.arange(end[i] - y[i], end[i] + 1) for i in range(n)])
        g.add_graph_node_properties(rows, np.zeros(rows.size, dtype=np.int64))
        if flip:
            wrong = rng.random(n) <= noise
            y = np.where(wrong, (y + rng.integers(1, classes, size=n)) % classes, y).astype(np.uint32)
        g.encode()
        return g, y

    gtr, ytr = build(n_train, None, True)
    gte, yte = build(n_test, gtr, False)
    params = dict(number_of_clauses=60, T=600, s=1.0, depth=3, message_size=256, message_bits=2,
                  max_included_literals=4)
    return Workload("runs_of_a", gtr, ytr, gte, yte, params, classes)


BUILDERS = {
    "noisy_xor": noisy_xor,
    "single_node_images": single_node_images,
    "convolutional_images": convolutional_images,
    "sequence_chains": sequence_chains,
    "colour_convolution": colour_convolution,
    "runs_of_a": runs_of_a,
}
