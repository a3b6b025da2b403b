"""Host-side graph container and hypervector bit-encoder.

Drop-in for the reference's ``Graphs`` (GraphTsetlinMachine/graphs.py:26-305):
same constructor, same builder methods, same public arrays with the same
dtypes and memory layout, so that a script written against the reference
builds byte-identical ``X`` / ``edge`` / index arrays here.

Array layout (all ``uint32``; this is what the device kernels index):

``X[total_nodes][number_of_hypervector_chunks]``
    literal ``k < hypervector_size`` is the symbol bit ``k``; literal
    ``k + hypervector_size`` is its negation.  Every node starts with all
    negated literals set (graphs.py:91-98, 112-113); a property sets bit ``k``
    and clears bit ``k + hypervector_size`` for each hypervector index ``k``
    of the symbol (graphs.py:148-159).
``node_type[total_nodes]``, ``number_of_graph_node_edges[total_nodes]``
``edge[E][2]``
    ``(graph-local destination node, edge type id)`` (graphs.py:143-145);
    the out-edges of consecutive nodes are contiguous.
``node_index[g]``, ``edge_index[node]``
    exclusive prefix sums (graphs.py:101-102, 128).

On top of the per-call builder API this class offers bulk, vectorised
variants (``add_graph_nodes``, ``add_graph_node_edges``,
``add_graph_node_properties``) because workloads with 10^8..10^9 property
insertions cannot be built one Python call at a time.
"""

import ctypes
import hashlib
import os

import numpy as np

_ENCODER_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libgtm_encode.so")
_encoder = None


def _native_encoder():
    """The C encoder of csrc/encode.c (built by build.py), or None when it has not been built or
    GTM_NO_NATIVE_ENCODER is set: the NumPy forms below give the same arrays, more slowly."""
    global _encoder
    if os.environ.get("GTM_NO_NATIVE_ENCODER"):
        return None
    if _encoder is None:
        if not os.path.exists(_ENCODER_PATH):
            return None
        lib = ctypes.CDLL(_ENCODER_PATH)
        p, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
        lib.gtm_encode_membership.restype = None
        lib.gtm_encode_membership.argtypes = [p, i64, i32, p, i32, i32, i32, p]
        lib.gtm_encode_pairs.restype = None
        lib.gtm_encode_pairs.argtypes = [p, p, i64, p, i32, i32, i32, p]
        _encoder = lib
    return _encoder


class GraphsError(SystemExit):
    """Raised on builder misuse.

    The reference prints a message and calls ``sys.exit(-1)``
    (graphs.py:134-136, 215-218).  ``sys.exit`` raises ``SystemExit``; this
    subclass keeps that behaviour (exit status -1 when uncaught) while
    carrying the message for callers that want to catch it.
    """

    def __init__(self, message):
        super().__init__(-1)
        self.message = message

    def __str__(self):
        return self.message


def _as_index_array(values):
    return np.ascontiguousarray(np.asarray(values, dtype=np.int64).reshape(-1))


class Graphs:
    def __init__(
        self,
        number_of_graphs,
        hypervector_size=128,
        hypervector_bits=2,
        double_hashing=False,
        one_hot_encoding=False,
        symbols=None,
        init_with=None,
    ):
        self.number_of_graphs = number_of_graphs
        self.number_of_graph_nodes = np.zeros(number_of_graphs, dtype=np.uint32)
        self.double_hashing = double_hashing
        self.one_hot_encoding = one_hot_encoding
        self.graph_node_id = [dict() for _ in range(number_of_graphs)]
        self.init_with = init_with
        self.encoded = False

        if init_with is not None:
            # The vocabulary objects are shared, not copied (graphs.py:80-86):
            # a type first seen in a test set is appended to the same dict.
            self.edge_type_id = init_with.edge_type_id
            self.node_type_id = init_with.node_type_id
            self.symbol_id = init_with.symbol_id
            self.hypervector_size = init_with.hypervector_size
            self.hypervector_bits = init_with.hypervector_bits
            self.hypervectors = init_with.hypervectors
            self.number_of_hypervector_chunks = init_with.number_of_hypervector_chunks
            return

        self.edge_type_id = {}
        self.node_type_id = {}
        self.symbol_id = {}
        for name in symbols:
            self.symbol_id[name] = len(self.symbol_id)
        n_symbols = len(self.symbol_id)
        self.hypervector_size = hypervector_size
        self.hypervector_bits = hypervector_bits

        if one_hot_encoding:
            # graphs.py:58-63
            self.hypervector_size = n_symbols
            self.hypervector_bits = 1
            self.hypervectors = np.arange(n_symbols, dtype=np.uint32).reshape(n_symbols, 1)
        elif double_hashing:
            # graphs.py:64-71
            from sympy import prevprime

            self.hypervector_bits = 2
            prime = int(prevprime(self.hypervector_size))
            ids = np.arange(n_symbols, dtype=np.int64)
            self.hypervectors = np.stack(
                [ids % self.hypervector_size, prime - (ids % prime)], axis=1
            ).astype(np.uint32)
        else:
            # graphs.py:73-76: one draw per symbol, in symbol order, from the
            # global legacy NumPy generator, so np.random.seed reproduces the
            # table of a reference run.
            self.hypervectors = np.zeros((n_symbols, self.hypervector_bits), dtype=np.uint32)
            indexes = np.arange(self.hypervector_size)
            for i in range(n_symbols):
                self.hypervectors[i, :] = np.random.choice(
                    indexes, size=(self.hypervector_bits), replace=False
                )

        self.number_of_hypervector_chunks = (self.hypervector_size * 2 - 1) // 32 + 1

    # ------------------------------------------------------------------ nodes

    def set_number_of_graph_nodes(self, graph_id, number_of_graph_nodes):
        self.number_of_graph_nodes[graph_id] = number_of_graph_nodes

    def _blank_rows(self, n_rows):
        """Rows with no property: positive half 0, negated half 1, padding 0."""
        hv = self.hypervector_size
        lit = np.arange(self.number_of_hypervector_chunks * 32, dtype=np.int64).reshape(-1, 32)
        negated = (lit >= hv) & (lit < 2 * hv)
        row = (negated.astype(np.uint64) << np.arange(32, dtype=np.uint64)).sum(axis=1)
        rows = np.empty((n_rows, row.shape[0]), dtype=np.uint32)
        rows[:] = row.astype(np.uint32)  # (a broadcast store: np.tile goes through repeat, ten times slower)
        return rows

    def prepare_node_configuration(self):
        counts = self.number_of_graph_nodes
        self.node_index = np.zeros(counts.shape[0], dtype=np.uint32)
        self.node_index[1:] = np.add.accumulate(counts[:-1])
        self.max_number_of_graph_nodes = counts.max()
        # 0 for a data set without nodes (the reference's unsigned subtraction wraps there, graphs.py:105)
        self.max_number_of_graph_node_chunks = np.uint32((int(self.max_number_of_graph_nodes) - 1) // 32 + 1)
        self.number_of_nodes = counts.sum()
        n = int(self.number_of_nodes)
        self.node_type = np.empty(n, dtype=np.uint32)
        self.number_of_graph_node_edges = np.empty(n, dtype=np.uint32)
        self.graph_node_edge_counter = np.zeros(n, dtype=np.uint32)
        self.edge_index = np.zeros(n, dtype=np.uint32)
        self.X = self._blank_rows(n)

    def _node_type(self, node_type_name):
        if node_type_name not in self.node_type_id:
            self.node_type_id[node_type_name] = len(self.node_type_id)
        return self.node_type_id[node_type_name]

    def add_graph_node(self, graph_id, node_name, number_of_graph_node_edges, node_type_name="Plain"):
        type_id = self._node_type(node_type_name)
        names = self.graph_node_id[graph_id]
        if node_name not in names:
            if isinstance(names, _RangeNames):
                # a name outside 0..n-1 after the bulk builder: fall back to the reference's dict
                names = self.graph_node_id[graph_id] = dict(names.items())
            names[node_name] = len(names)
        row = int(self.node_index[graph_id]) + names[node_name]
        self.node_type[row] = type_id
        self.number_of_graph_node_edges[row] = number_of_graph_node_edges

    def add_graph_nodes(self, number_of_graph_node_edges, node_type_name="Plain", node_types=None):
        """Bulk form of ``add_graph_node`` for every node of every graph.

        Nodes of graph ``g`` are named ``0 .. number_of_graph_nodes[g]-1`` (as
        in the reference's sequence and image demos) and get local ids in that
        order.  ``number_of_graph_node_edges`` is an array over all nodes in
        ``node_index`` order (or a scalar).  ``node_types`` optionally gives a
        per-node array of node type *names*; otherwise every node gets
        ``node_type_name``.
        """
        n = int(self.number_of_nodes)
        for g in range(self.number_of_graphs):
            count = int(self.number_of_graph_nodes[g])
            self.graph_node_id[g] = _RangeNames(count)
        if node_types is None:
            self.node_type[:] = self._node_type(node_type_name)
        else:
            node_types = np.asarray(node_types).reshape(-1)
            if node_types.shape[0] != n:
                raise ValueError("node_types must have one entry per node")
            ids = np.empty(n, dtype=np.uint32)
            for name in dict.fromkeys(node_types.tolist()):
                ids[node_types == name] = self._node_type(name)
            self.node_type[:] = ids
        self.number_of_graph_node_edges[:] = np.broadcast_to(
            np.asarray(number_of_graph_node_edges, dtype=np.uint32), (n,)
        )

    def number_of_node_types(self):
        return len(self.node_type_id)

    # ------------------------------------------------------------------ edges

    def prepare_edge_configuration(self):
        self.edge_index[1:] = np.add.accumulate(self.number_of_graph_node_edges[:-1])
        self.edge = np.empty((int(self.number_of_graph_node_edges.sum()), 2), dtype=np.uint32)

    def _edge_type(self, edge_type_name):
        if edge_type_name not in self.edge_type_id:
            self.edge_type_id[edge_type_name] = len(self.edge_type_id)
        return self.edge_type_id[edge_type_name]

    def add_graph_node_edge(self, graph_id, source_node_name, destination_node_name, edge_type_name):
        names = self.graph_node_id[graph_id]
        row = int(self.node_index[graph_id]) + names[source_node_name]
        used = int(self.graph_node_edge_counter[row])
        if used >= int(self.number_of_graph_node_edges[row]):
            message = "Too many edges added to node '%s' of graph %d." % (source_node_name, graph_id)
            print(message)
            raise GraphsError(message)
        destination = names[destination_node_name]
        type_id = self._edge_type(edge_type_name)
        slot = int(self.edge_index[row]) + used
        self.edge[slot, 0] = destination
        self.edge[slot, 1] = type_id
        self.graph_node_edge_counter[row] = used + 1

    def add_graph_node_edges(self, graph_ids, source_nodes, destination_nodes, edge_type_names):
        """Bulk form of ``add_graph_node_edge``.

        ``source_nodes`` / ``destination_nodes`` are graph-local node ids.
        Edges are appended to each source node in the order given, exactly as
        the same sequence of single calls would.  ``edge_type_names`` is one
        name or a sequence of names (one per edge); type ids are assigned in
        order of first appearance.
        """
        graph_ids = _as_index_array(graph_ids)
        src = _as_index_array(source_nodes)
        dst = _as_index_array(destination_nodes)
        n_edges = src.shape[0]
        if isinstance(edge_type_names, (str, bytes)) or np.isscalar(edge_type_names):
            type_ids = np.full(n_edges, self._edge_type(edge_type_names), dtype=np.uint32)
        else:
            names = np.asarray(edge_type_names).reshape(-1)
            type_ids = np.empty(n_edges, dtype=np.uint32)
            for name in dict.fromkeys(names.tolist()):
                type_ids[names == name] = self._edge_type(name)
        counts = self.number_of_graph_nodes[graph_ids].astype(np.int64)
        if ((src < 0) | (src >= counts) | (dst < 0) | (dst >= counts)).any():
            raise IndexError("edge endpoint outside its graph")
        rows = self.node_index[graph_ids].astype(np.int64) + src
        # rank of each edge among the edges of its source row, in call order
        order = np.argsort(rows, kind="stable")
        sorted_rows = rows[order]
        first = np.r_[0, np.flatnonzero(np.diff(sorted_rows)) + 1]
        run_start = np.repeat(first, np.diff(np.r_[first, n_edges]))
        rank = np.empty(n_edges, dtype=np.int64)
        rank[order] = np.arange(n_edges) - run_start
        used = self.graph_node_edge_counter[rows].astype(np.int64) + rank
        over = used >= self.number_of_graph_node_edges[rows].astype(np.int64)
        if over.any():
            bad = int(np.flatnonzero(over)[0])
            message = "Too many edges added to node '%s' of graph %d." % (src[bad], graph_ids[bad])
            print(message)
            raise GraphsError(message)
        slots = self.edge_index[rows].astype(np.int64) + used
        self.edge[slots, 0] = dst
        self.edge[slots, 1] = type_ids
        np.add.at(self.graph_node_edge_counter, rows, 1)

    # ------------------------------------------------------------- properties

    def add_graph_node_property(self, graph_id, node_name, symbol):
        row = int(self.node_index[graph_id]) + self.graph_node_id[graph_id][node_name]
        hv = self.hypervector_size
        x = self.X[row]
        for k in self.hypervectors[self.symbol_id[symbol], :]:
            k = int(k)
            x[k >> 5] |= np.uint32(1 << (k & 31))
            n = k + hv
            x[n >> 5] &= np.uint32(~(1 << (n & 31)) & 0xFFFFFFFF)

    def _encodable(self):
        """The arrays are as the C encoder addresses them: contiguous uint32, every hypervector index
        inside the hypervector."""
        return (self.X.dtype == np.uint32 and self.X.flags.c_contiguous and self.hypervectors.dtype == np.uint32 and
                self.hypervectors.flags.c_contiguous and self.hypervectors.ndim == 2 and
                (self.hypervectors.size == 0 or int(self.hypervectors.max()) < self.hypervector_size))

    def add_graph_node_properties(self, node_rows, symbol_ids, chunk_rows=1 << 18):
        """Bulk form of ``add_graph_node_property``.

        ``node_rows`` are global node rows (``node_index[g] + local id``) and
        ``symbol_ids`` the matching ``symbol_id`` values; pair ``i`` adds symbol
        ``symbol_ids[i]`` to node ``node_rows[i]``.  Setting a bit is
        idempotent, so the pairs may repeat and come in any order.
        """
        rows = _as_index_array(node_rows)
        syms = _as_index_array(symbol_ids)
        if rows.shape != syms.shape:
            raise ValueError("node_rows and symbol_ids must have the same length")
        if rows.size == 0:
            return
        if rows.min() < 0 or rows.max() >= self.X.shape[0] or syms.min() < 0 or syms.max() >= self.hypervectors.shape[0]:
            raise IndexError("node row or symbol id out of range")
        native = _native_encoder()
        if native is not None and self._encodable():
            native.gtm_encode_pairs(rows.ctypes.data, syms.ctypes.data, rows.size, self.hypervectors.ctypes.data,
                                    self.hypervectors.shape[1], self.hypervector_size,
                                    self.number_of_hypervector_chunks, self.X.ctypes.data)
            return
        hv = self.hypervector_size
        chunks = self.number_of_hypervector_chunks
        order = np.argsort(rows, kind="stable")
        rows, syms = rows[order], syms[order]
        lo_row, hi_row = int(rows[0]), int(rows[-1]) + 1
        for start in range(lo_row, hi_row, chunk_rows):
            stop = min(start + chunk_rows, hi_row)
            a, b = np.searchsorted(rows, [start, stop])
            if a == b:
                continue
            positive = np.zeros((stop - start, hv), dtype=np.uint8)
            local = rows[a:b] - start
            for j in range(self.hypervector_bits):
                positive[local, self.hypervectors[syms[a:b], j]] = 1
            touched = np.unique(local)
            bits = np.zeros((touched.shape[0], chunks * 32), dtype=np.uint8)
            bits[:, :hv] = positive[touched]
            bits[:, hv : 2 * hv] = 1 - positive[touched]
            words = np.packbits(bits, axis=1, bitorder="little").view("<u4")
            # merge with what is already there: set positive bits, clear negated ones
            old = self.X[start + touched]
            blank = self._blank_rows(1)[0]
            pos_mask = ~blank
            new_pos = (old | words) & pos_mask
            new_neg = (old & words) & blank
            self.X[start + touched] = new_pos | new_neg

    def add_graph_node_property_matrix(self, first_node_row, membership, chunk_rows=1 << 16):
        """Bulk form of ``add_graph_node_property`` from a dense table.

        ``membership[r][s]`` non-zero adds the symbol with id ``s`` to node row
        ``first_node_row + r``.  The node rows are OR-ed with what they already
        hold, as repeated single calls would.
        """
        membership = np.asarray(membership)
        n_rows, n_symbols = membership.shape
        if n_symbols != len(self.symbol_id):
            raise ValueError("membership needs one column per symbol")
        if first_node_row < 0 or first_node_row + n_rows > self.X.shape[0]:
            raise IndexError("node rows out of range")
        native = _native_encoder()
        if native is not None and self._encodable() and n_rows > 0:
            flags = np.ascontiguousarray(membership if membership.dtype == np.uint8 else membership != 0).view(np.uint8)
            target = self.X[first_node_row:first_node_row + n_rows]
            native.gtm_encode_membership(flags.ctypes.data, n_rows, n_symbols, self.hypervectors.ctypes.data,
                                         self.hypervectors.shape[1], self.hypervector_size,
                                         self.number_of_hypervector_chunks, target.ctypes.data)
            return
        hv = self.hypervector_size
        chunks = self.number_of_hypervector_chunks
        # symbol -> hypervector index incidence; small-integer float32 products are exact
        incidence = np.zeros((n_symbols, hv), dtype=np.float32)
        for j in range(self.hypervector_bits):
            incidence[np.arange(n_symbols), self.hypervectors[:, j]] = 1.0
        blank = self._blank_rows(1)[0]
        for start in range(0, n_rows, chunk_rows):
            stop = min(start + chunk_rows, n_rows)
            positive = (membership[start:stop].astype(np.float32) @ incidence) > 0.0
            bits = np.zeros((stop - start, chunks * 32), dtype=np.uint8)
            bits[:, :hv] = positive
            bits[:, hv : 2 * hv] = ~positive
            words = np.packbits(bits, axis=1, bitorder="little").view("<u4")
            rows = slice(first_node_row + start, first_node_row + stop)
            old = self.X[rows]
            self.X[rows] = ((old | words) & ~blank) | (old & words & blank)

    # ------------------------------------------------------------------ print

    def print_graph_nodes(self, graph_id):
        text = "Printing nodes of Graph#" + str(graph_id) + ":\n"
        base = int(self.node_index[graph_id])
        for node_id in range(int(self.number_of_graph_nodes[graph_id])):
            row = self.X[base + node_id]
            text += "Node#" + str(node_id) + "( "
            for symbol_name, symbol_id in self.symbol_id.items():
                ks = self.hypervectors[symbol_id, :].astype(np.int64)
                present = bool(np.all((row[ks >> 5] >> (ks & 31).astype(np.uint32)) & 1))
                text += (str(symbol_name) if present else "*") + " "
            text += ") "
        print(text)
        print()

    def print_graph_edges(self, graph_id):
        text = "Printing edges of Graph#" + str(graph_id) + ":\n"
        base = int(self.node_index[graph_id])
        for node_id in range(int(self.number_of_graph_nodes[graph_id])):
            for j in range(int(self.graph_node_edge_counter[base + node_id])):
                slot = int(self.edge_index[base + node_id]) + j
                text += "Edge#%d SrcNode#%d DestNode#%d EdgeType#%d\n" % (
                    slot,
                    node_id,
                    self.edge[slot][0],
                    self.edge[slot][1],
                )
            text += "\n"
        print(text)
        print()

    def print_graph(self, graph_id):
        self.print_graph_nodes(graph_id)
        self.print_graph_edges(graph_id)

    # ----------------------------------------------------------------- encode

    def encode(self):
        """Check that every declared edge was added and fingerprint the data
        (graphs.py:209-225): ``signature = sha256(X || edge)``."""
        missing = np.flatnonzero(self.graph_node_edge_counter < self.number_of_graph_node_edges)
        if missing.size:
            owner = np.searchsorted(self.node_index, missing, side="right") - 1
            lines = []
            for row, g in zip(missing.tolist(), owner.tolist()):
                local = row - int(self.node_index[g])
                name = local
                for node_name, node_id in self.graph_node_id[g].items():
                    if node_id == local:
                        name = node_name
                        break
                lines.append("Node '%s' of graph %d misses edges." % (name, g))
            print("\n".join(lines))
            raise GraphsError("\n".join(lines))
        m = hashlib.sha256()
        m.update(np.ascontiguousarray(self.X).data)
        m.update(np.ascontiguousarray(self.edge).data)
        self.signature = m.digest()
        self.encoded = True

    # -------------------------------------------------------------- subsetting

    def __len__(self):
        return self.number_of_graphs

    def _get_indices(self, key):
        if isinstance(key, (int, np.integer)):
            key = [int(key)]
        elif isinstance(key, slice):
            return list(range(*key.indices(self.number_of_graphs)))
        elif not isinstance(key, (list, np.ndarray)):
            raise TypeError("Invalid graph index type")
        indices = []
        for k in key:
            k = int(k)
            if k < 0:
                k += self.number_of_graphs
            if k < 0 or k >= self.number_of_graphs:
                raise IndexError("Graph index out of range")
            indices.append(k)
        return indices

    def __getitem__(self, index):
        """A new, encoded ``Graphs`` holding the selected graphs
        (graphs.py:231-305), sharing vocabulary and hypervectors."""
        indices = self._get_indices(index)
        if len(indices) == 0:
            raise ValueError("No graphs selected")
        picked = np.asarray(indices, dtype=np.int64)
        subset = Graphs(
            len(indices),
            double_hashing=self.double_hashing,
            one_hot_encoding=self.one_hot_encoding,
            init_with=self,
        )
        subset.number_of_graph_nodes[:] = self.number_of_graph_nodes[picked]
        subset.graph_node_id = [self.graph_node_id[g] for g in indices]
        subset.prepare_node_configuration()

        counts = self.number_of_graph_nodes[picked].astype(np.int64)
        starts = self.node_index[picked].astype(np.int64)
        within = np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)
        old_rows = np.repeat(starts, counts) + within
        subset.node_type[:] = self.node_type[old_rows]
        subset.number_of_graph_node_edges[:] = self.number_of_graph_node_edges[old_rows]
        subset.graph_node_edge_counter[:] = self.graph_node_edge_counter[old_rows]
        subset.X[:] = self.X[old_rows]
        subset.prepare_edge_configuration()

        # per node the edges added so far (graphs.py:288-296 copies graph_node_edge_counter of them);
        # for a complete data set that is every declared edge
        e_counts = self.graph_node_edge_counter[old_rows].astype(np.int64)
        e_starts = self.edge_index[old_rows].astype(np.int64)
        e_within = np.arange(int(e_counts.sum())) - np.repeat(np.cumsum(e_counts) - e_counts, e_counts)
        if int(e_counts.sum()) != subset.edge.shape[0]:
            subset.edge[:] = 0  # slots of edges not yet added (encode() below reports them)
        new_starts = subset.edge_index.astype(np.int64)
        subset.edge[np.repeat(new_starts, e_counts) + e_within] = self.edge[np.repeat(e_starts, e_counts) + e_within]
        subset.encode()
        return subset


class _RangeNames:
    """Mapping ``name -> local id`` for nodes named ``0..n-1`` without
    materialising a dict per graph (bulk builder)."""

    __slots__ = ("n",)

    def __init__(self, n):
        self.n = n

    def __getitem__(self, name):
        i = int(name)
        if i < 0 or i >= self.n:
            raise KeyError(name)
        return i

    def __contains__(self, name):
        try:
            i = int(name)
        except (TypeError, ValueError):
            return False
        return 0 <= i < self.n

    def __len__(self):
        return self.n

    def items(self):
        return ((i, i) for i in range(self.n))
