"""Graph Tsetlin Machine models on the HIP hot path.

Host-side mirror of the reference's ``CommonTsetlinMachine`` and its public
subclasses (GraphTsetlinMachine/tm.py:38-1072): same constructor arguments,
same ``fit / score / predict / get_state / save / load / ta_action /
get_weights`` and the same state layouts, so pickles made by ``save`` carry
the reference's 24 keys with the reference's array shapes and dtypes.

What differs underneath: the per-graph Python loop with a device
synchronisation after every launch (tm.py:563-747, 786-812) is replaced by
one C-ABI call per ``fit`` epoch / per ``score`` (``gtm_fit`` / ``gtm_score``),
torch tensors only own the device memory, and random decisions come from a
counter-based generator keyed by ``seed`` (argument added at the end of the
constructor; drawn from NumPy's global generator when omitted, so
``np.random.seed`` still makes runs repeatable).  ``grid`` and ``block`` are
accepted and ignored: launch shapes are chosen by the library.
"""

import ctypes
import io
import os
import pickle
import sys

import numpy as np
import torch

from . import _abi


def _device():
    if not torch.cuda.is_available():
        raise _abi.GtmError("no GPU visible: the Graph Tsetlin Machine hot path runs on the HIP device only")
    return torch.device("cuda", torch.cuda.current_device())


def _to_device(array):
    """uint32/int32 NumPy array -> int32 torch tensor on the GPU (same bits)."""
    a = np.ascontiguousarray(array)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a.reshape(-1)).to(_device())


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else ctypes.c_void_p(0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class _DeviceGraphs:
    """Device copy of a Graphs object's arrays (tm.py:528-555, 759-784)."""

    def __init__(self, graphs):
        self.signature = graphs.signature
        self.number_of_graphs = int(graphs.number_of_graphs)
        self.max_nodes = int(graphs.max_number_of_graph_nodes)
        self.tensors = {
            "X": _to_device(graphs.X),
            "node_type": _to_device(graphs.node_type),
            "number_of_graph_node_edges": _to_device(graphs.number_of_graph_node_edges),
            "edge": _to_device(graphs.edge),
            "node_index": _to_device(graphs.node_index),
            "edge_index": _to_device(graphs.edge_index),
            "number_of_graph_nodes": _to_device(graphs.number_of_graph_nodes),
        }
        d = _abi.GraphsDesc()
        for name, t in self.tensors.items():
            setattr(d, name, _ptr(t))
        d.number_of_graphs = self.number_of_graphs
        d.number_of_node_types = graphs.number_of_node_types()
        d.max_number_of_graph_nodes = self.max_nodes
        d.total_nodes = int(graphs.number_of_nodes)
        d.total_edges = int(graphs.edge.shape[0])
        d.tiles = None
        self.desc = d
        self.tiles = None
        self._tiles_key = None
        self._complementary = None  # not looked at yet

    def ensure_tiles(self, cfg):
        """Build the literal-major tile layout once per data set and tile
        geometry (used by inference and training); shapes without such a
        layout keep tiles = NULL.  The geometry depends on the model's
        sizes, so a data set handed to a model of another shape is tiled
        again."""
        key = (cfg.classes, cfg.literals, cfg.depth, cfg.message_size, _abi.tuning("GTM_TILE_LANE_WORDS"),
               _abi.tuning("GTM_NO_HALF_TILES"), _abi.tuning("GTM_NO_TWO_PHASE"), _abi.tuning("GTM_HALF_LANE_WORDS"))
        if self._tiles_key == key:
            return
        self._tiles_key = key
        self.tiles = None
        self.desc.tiles = None
        if self._complementary is None and cfg.literals % 2 == 0:
            # one look at the data on the device: are the negated literals the complements of the
            # positive ones everywhere, and has every graph a node?  (What Graphs builds - but X is a
            # public array.)  Then the tile kernels may keep half the rows on chip.
            found = torch.zeros(2, dtype=torch.int32, device=_device())
            _abi.call("gtm_graphs_properties", ctypes.byref(cfg), ctypes.byref(self.desc), _ptr(found), _stream())
            self._complementary = not found.cpu().numpy().any()
        self.desc.flags = _abi.GTM_GRAPHS_COMPLEMENTARY if self._complementary else 0
        nbytes = _abi.lib.gtm_tiles_bytes(ctypes.byref(cfg), ctypes.byref(self.desc))
        if nbytes == 0:
            return
        self.tiles = torch.empty(nbytes // 4, dtype=torch.int32, device=_device())
        _abi.call("gtm_build_tiles", ctypes.byref(cfg), ctypes.byref(self.desc), _ptr(self.tiles), _stream())
        self.desc.tiles = self.tiles.data_ptr()


class ModelState(tuple):
    """The 10-tuple of ``get_state`` (tm.py:287) with the message banks riding
    along as an attribute; indexes, unpacks and compares as the plain tuple."""

    message_ta_state = None


_NPZ_ARRAYS = ("ta_state", "clause_weights", "hypervectors")
_NPZ_SCALARS = (
    "number_of_outputs", "number_of_literals", "number_of_message_literals", "min_y", "max_y", "negative_clauses",
    "max_number_of_graph_nodes", "number_of_clauses", "T", "q", "max_included_literals",
    "boost_true_positive_feedback", "number_of_state_bits", "depth", "message_size", "message_bits",
    "double_hashing", "one_hot_encoding", "rng_seed", "rng_step",
)


class _StateUnpickler(pickle.Unpickler):
    """Reads the dict that ``save`` pickles (tm.py:328-356: NumPy arrays, NumPy and Python scalars,
    tuples, lists) and nothing else: a pickle may name any importable callable and have it run
    while it loads, so every global it asks for is checked against the few that rebuild arrays
    and scalars, and anything else ends the load before it runs."""

    _ALLOWED = {
        ("numpy", "ndarray"), ("numpy", "dtype"),
        ("numpy.core.multiarray", "_reconstruct"), ("numpy._core.multiarray", "_reconstruct"),
        ("numpy.core.multiarray", "scalar"), ("numpy._core.multiarray", "scalar"),
        ("numpy.core.numeric", "_frombuffer"), ("numpy._core.numeric", "_frombuffer"),
        ("builtins", "dict"), ("builtins", "tuple"), ("builtins", "list"), ("builtins", "int"),
        ("builtins", "float"), ("builtins", "bool"), ("builtins", "complex"), ("builtins", "bytes"),
        ("builtins", "str"), ("builtins", "bytearray"),
    }

    def find_class(self, module, name):
        if (module, name) not in self._ALLOWED:
            raise pickle.UnpicklingError(
                "the state file asks for %s.%s: only NumPy arrays, scalars and plain containers are loaded"
                % (module, name))
        return super().find_class(module, name)


def read_state_pickle(fname):
    """The dict of a ``save(fname)`` pickle - this class's or the reference's (tm.py:356-357) - read
    without running anything the file names."""
    with open(fname, "rb") as f:
        state_dict = _StateUnpickler(io.BytesIO(f.read())).load()
    if not isinstance(state_dict, dict):
        raise pickle.UnpicklingError("the state file holds a %s, not the dict that save() writes" % type(state_dict).__name__)
    return state_dict


def write_state_npz(state_dict, fname):
    """The dict of ``save`` (tm.py:328-354) as a NumPy archive of plain arrays:
    nothing in it is pickled, so ``numpy.load(allow_pickle=False)`` reads it.
    Message banks become ``message_ta_state_<i>``, ``s`` a float array, scalars
    0-d arrays; a value of None is left out."""
    out = {name: np.asarray(state_dict[name]) for name in _NPZ_ARRAYS}
    for i, bank in enumerate(state_dict["message_ta_state"]):
        out["message_ta_state_%d" % i] = np.asarray(bank, dtype=np.uint32)
    out["s"] = np.asarray(state_dict["s"], dtype=np.float64).reshape(-1)
    for name in _NPZ_SCALARS:
        value = state_dict.get(name)
        if value is None:
            continue
        out[name] = np.asarray(value, dtype=np.uint64 if name == "rng_seed" else None)
    with open(fname, "wb") as f:
        np.savez(f, **out)


def read_state_npz(fname):
    """Inverse of ``write_state_npz``: the dict ``load`` takes."""
    with np.load(fname, allow_pickle=False) as z:
        d = {name: z[name] for name in _NPZ_ARRAYS}
        banks = []
        while "message_ta_state_%d" % len(banks) in z.files:
            banks.append(z["message_ta_state_%d" % len(banks)])
        d["message_ta_state"] = banks
        d["s"] = tuple(float(v) for v in z["s"])
        for name in _NPZ_SCALARS:
            if name not in z.files:
                if name not in ("rng_seed", "rng_step"):
                    d[name] = None
                continue
            v = z[name][()]
            if name in ("double_hashing", "one_hot_encoding"):
                d[name] = bool(v)
            elif name == "q":
                d[name] = float(v)
            else:
                d[name] = int(v)
    return d


class CommonTsetlinMachine:
    def __init__(
        self,
        number_of_clauses,
        T,
        s,
        q=1.0,
        max_included_literals=None,
        boost_true_positive_feedback=1,
        number_of_state_bits=8,
        depth=1,
        message_size=256,
        message_bits=2,
        double_hashing=False,
        one_hot_encoding=False,
        grid=(16 * 13 * 4, 1, 1),
        block=(128, 1, 1),
        seed=None,
    ):
        self.number_of_clauses = number_of_clauses
        self.number_of_clause_chunks = (number_of_clauses - 1) // 32 + 1
        self.T = int(T)
        self.depth = depth
        self.s = s if type(s) == tuple else (s,) * self.depth  # tm.py:63-66
        self.q = q
        self.max_included_literals = max_included_literals
        self.boost_true_positive_feedback = boost_true_positive_feedback
        self.number_of_state_bits = number_of_state_bits
        self.message_size = message_size
        self.message_bits = message_bits
        self.double_hashing = double_hashing
        self.one_hot_encoding = one_hot_encoding
        self.grid = grid
        self.block = block

        self.graphs_signature_train = np.array([])
        self.graphs_signature_test = np.array([])
        self.encoded_Y = np.array([])
        self.ta_state = np.array([])
        self.message_ta_state = [np.array([])] * (self.depth - 1)
        self.clause_weights = np.array([])

        # Clause message hypervectors (tm.py:90-106): which message bits a
        # true clause sets at its neighbours.
        if self.one_hot_encoding:
            self.message_bits = 1
            self.hypervectors = np.zeros((number_of_clauses, 1), dtype=np.uint32)  # filled in _init
        elif self.double_hashing:
            from sympy import prevprime

            self.message_bits = 2
            prime = int(prevprime(self.message_size))
            ids = np.arange(number_of_clauses, dtype=np.int64)
            self.hypervectors = np.stack([ids % self.message_size, prime - (ids % prime)], axis=1).astype(np.uint32)
        else:
            indexes = np.arange(self.message_size, dtype=np.uint32)
            self.hypervectors = np.zeros((number_of_clauses, self.message_bits), dtype=np.uint32)
            for i in range(number_of_clauses):
                self.hypervectors[i, :] = np.random.choice(indexes, size=(self.message_bits), replace=False)

        if seed is None:
            seed = int(np.random.randint(0, 2**32, dtype=np.uint64)) | (int(np.random.randint(0, 2**32, dtype=np.uint64)) << 32)
        self.seed = int(seed)
        self.step = 0  # training examples seen so far; addresses the random draws

        self.initialized = False
        self._train_graphs = None
        self._test_graphs = None
        self._workspace = None
        self._encoded_Y_gpu = None

    # ------------------------------------------------------------ sizing

    def _init(self, graphs):
        """tm.py:414-435."""
        if self.one_hot_encoding:
            n_edge_types = len(graphs.edge_type_id)
            self.message_size = self.number_of_clauses * max(1, n_edge_types)
            self.hypervectors[:, 0] = np.arange(self.number_of_clauses) * n_edge_types
        self.number_of_features = graphs.hypervector_size
        self.number_of_literals = self.number_of_features * 2
        self.number_of_ta_chunks = int((self.number_of_literals - 1) // 32 + 1)
        self.number_of_message_features = self.message_size
        self.number_of_message_literals = self.number_of_message_features * 2
        self.number_of_message_chunks = int((self.number_of_message_literals - 1) // 32 + 1)
        if self.max_included_literals is None:
            self.max_included_literals = self.number_of_literals
        self.max_number_of_graph_nodes = graphs.max_number_of_graph_nodes
        self._allocate()
        self.initialized = True

    def _allocate(self):
        """tm.py:110-124."""
        dev = _device()
        C, B = self.number_of_clauses, self.number_of_state_bits
        self.ta_state_gpu = torch.empty(C * self.number_of_ta_chunks * B, dtype=torch.int32, device=dev)
        self.message_ta_state_gpu = [
            torch.empty(C * self.number_of_message_chunks * B, dtype=torch.int32, device=dev)
            for _ in range(self.depth - 1)
        ]
        self.clause_weights_gpu = torch.empty(self.number_of_outputs * C, dtype=torch.int32, device=dev)
        self._allocated_outputs = int(self.number_of_outputs)
        self.hypervectors_gpu = _to_device(self.hypervectors)
        st = _abi.State()
        st.ta_state = _ptr(self.ta_state_gpu)
        for i, t in enumerate(self.message_ta_state_gpu):
            st.message_ta_state[i] = t.data_ptr()
        st.clause_weights = _ptr(self.clause_weights_gpu)
        st.hypervectors = _ptr(self.hypervectors_gpu)
        self._state = st

    def _outputs_for(self, seen):
        """Number of outputs for a ``fit`` whose labels show ``seen`` of them.

        The weight buffer and the tile geometry are sized for the outputs of
        the first ``fit`` (the reference compiles CLASSES in then,
        tm.py:452).  A later batch may hold fewer labels - the model keeps
        its size - but never more: that would index past the buffers."""
        allocated = getattr(self, "_allocated_outputs", None)
        if not self.initialized or allocated is None:
            return int(seen)
        if seen > allocated:
            raise _abi.GtmError(
                "this model was sized for %d outputs at its first fit; the labels passed now need %d"
                % (allocated, seen)
            )
        return allocated

    def _config(self, max_nodes):
        if getattr(self, "_allocated_outputs", self.number_of_outputs) != self.number_of_outputs:
            raise _abi.GtmError(
                "number_of_outputs=%d differs from the %d outputs the device buffers were allocated for"
                % (self.number_of_outputs, self._allocated_outputs)
            )
        return _abi.make_config(
            classes=self.number_of_outputs,
            clauses=self.number_of_clauses,
            literals=self.number_of_literals,
            state_bits=self.number_of_state_bits,
            boost_true_positive_feedback=self.boost_true_positive_feedback,
            threshold=self.T,
            q=self.q,
            max_included_literals=self.max_included_literals,
            negative_clauses=self.negative_clauses,
            max_nodes=int(max_nodes),
            message_size=self.message_size,
            message_bits=self.message_bits,
            depth=self.depth,
            s=self.s,
            seed=self.seed,
        )

    def _workspace_of(self, nbytes):
        if self._workspace is None or self._workspace.numel() < nbytes:
            self._workspace = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=_device())
        return self._workspace

    # ------------------------------------------------------------- training

    def _prepare(self, cfg, with_message_banks):
        _abi.call("gtm_prepare", ctypes.byref(cfg), self.step, _ptr(self.ta_state_gpu), _ptr(self.clause_weights_gpu), _stream())
        if with_message_banks:
            for t in self.message_ta_state_gpu:
                _abi.call("gtm_prepare_message_ta_state", ctypes.byref(cfg), _ptr(t), _stream())

    def _init_fit(self, graphs, encoded_Y, incremental):
        """tm.py:515-561."""
        if not self.initialized:
            self._init(graphs)
            self._prepare(self._config(graphs.max_number_of_graph_nodes), True)
        elif incremental == False:  # noqa: E712  (the reference re-initialises layer 0 only, tm.py:524-526)
            self._prepare(self._config(graphs.max_number_of_graph_nodes), False)
        if self._train_graphs is None or not np.array_equal(self.graphs_signature_train, graphs.signature):
            self.graphs_signature_train = graphs.signature
            self._train_graphs = _DeviceGraphs(graphs)
        if self._encoded_Y_gpu is None or not np.array_equal(self.encoded_Y, encoded_Y):
            self.encoded_Y = encoded_Y
            self._encoded_Y_gpu = _to_device(np.ascontiguousarray(encoded_Y, dtype=np.int32))

    def _fit(self, graphs, encoded_Y, epochs=100, incremental=False, examples=None):
        """tm.py:664-752; each epoch is one gtm_fit call.  ``examples=(first, count)`` (not in
        the reference) restricts an epoch to that run of the data set's graphs, so that a
        resident data set can be trained on piece by piece without being cut up."""
        self._init_fit(graphs, encoded_Y, incremental)
        dg = self._train_graphs
        cfg = self._config(max(dg.max_nodes, 1))
        dg.ensure_tiles(cfg)
        need = _abi.lib.gtm_fit_workspace_bytes(ctypes.byref(cfg), ctypes.byref(dg.desc))
        ws = self._workspace_of(need)
        first, count = (0, dg.number_of_graphs) if examples is None else (int(examples[0]), int(examples[1]))
        if first < 0 or count < 0 or first + count > dg.number_of_graphs:
            raise _abi.GtmError("examples=(%d, %d) outside the data set's %d graphs" % (first, count, dg.number_of_graphs))
        for _ in range(epochs):
            _abi.call(
                "gtm_fit", ctypes.byref(cfg), ctypes.byref(dg.desc), ctypes.byref(self._state),
                _ptr(self._encoded_Y_gpu), first, count, self.step, _ptr(ws), ws.numel(), _stream(),
            )
            self.step += count
        torch.cuda.current_stream().synchronize()
        self.ta_state = np.array([])
        self.clause_weights = np.array([])

    # ------------------------------------------------------------ inference

    def _score_init(self, graphs):
        """tm.py:754-784."""
        if not self.initialized:
            print("Error: Model not trained.")
            sys.exit(-1)
        if self._train_graphs is not None and np.array_equal(self.graphs_signature_train, graphs.signature):
            return self._train_graphs  # same data already resident
        if self._test_graphs is None or not np.array_equal(self.graphs_signature_test, graphs.signature):
            self.graphs_signature_test = graphs.signature
            self._test_graphs = _DeviceGraphs(graphs)
        return self._test_graphs

    def _score(self, graphs, batch=None):
        """tm.py:786-812 as one gtm_score call."""
        n = int(graphs.number_of_graphs)
        return self.score_device(graphs, batch).cpu().numpy().reshape(n, self.number_of_outputs)

    def score_device(self, graphs, batch=None):
        """Class sums as a flat int32 device tensor [graphs * outputs]; work is
        only enqueued on the current stream."""
        dg = self._score_init(graphs)
        cfg = self._config(max(dg.max_nodes, 1))
        n = dg.number_of_graphs
        dg.ensure_tiles(cfg)
        if batch is None:
            # as many graphs per launch group as fit in 4 GiB of workspace beyond its fixed part
            size = lambda b: _abi.lib.gtm_score_workspace_bytes(ctypes.byref(cfg), ctypes.byref(dg.desc), b)
            fixed = size(1)
            per_graph = max(1.0, (size(1025) - fixed) / 1024.0)
            batch = int(max(1, min(n, ((4 << 30) - fixed) // per_graph, 1 << 16)))
        need = _abi.lib.gtm_score_workspace_bytes(ctypes.byref(cfg), ctypes.byref(dg.desc), batch)
        ws = self._workspace_of(need)
        out = torch.empty(n * self.number_of_outputs, dtype=torch.int32, device=_device())
        _abi.call(
            "gtm_score", ctypes.byref(cfg), ctypes.byref(dg.desc), ctypes.byref(self._state), 0, n, batch,
            _ptr(ws), ws.numel(), _ptr(out), _stream(),
        )
        return out

    def _transform(self, graphs, nodewise, batch=None):
        """tm.py:814-900 as one gtm_transform call."""
        dg = self._score_init(graphs)
        cfg = self._config(max(dg.max_nodes, 1))
        n, C = dg.number_of_graphs, self.number_of_clauses
        dg.ensure_tiles(cfg)
        width = max(int(np.max(graphs.number_of_graph_nodes)), 1) if nodewise else 0
        if batch is None:
            size = lambda b: _abi.lib.gtm_transform_workspace_bytes(ctypes.byref(cfg), ctypes.byref(dg.desc), b)
            fixed = size(1)
            per_graph = max(1.0, (size(1025) - fixed) / 1024.0)
            batch = int(max(1, min(n, ((1 << 30) - fixed) // per_graph, 1 << 16)))
        need = _abi.lib.gtm_transform_workspace_bytes(ctypes.byref(cfg), ctypes.byref(dg.desc), batch)
        ws = self._workspace_of(need)
        sums = torch.empty(n * self.number_of_outputs, dtype=torch.int32, device=_device())
        flat = torch.empty(n * C, dtype=torch.int32, device=_device())
        wide = torch.empty(n * C * width, dtype=torch.int32, device=_device()) if nodewise else None
        _abi.call(
            "gtm_transform", ctypes.byref(cfg), ctypes.byref(dg.desc), ctypes.byref(self._state), 0, n, batch,
            _ptr(ws), ws.numel(), _ptr(flat), _ptr(wide) if nodewise else None, width, _ptr(sums), _stream(),
        )
        out = wide.cpu().numpy().reshape(n, C, width) if nodewise else flat.cpu().numpy().reshape(n, C)
        return out, sums.cpu().numpy().reshape(n, self.number_of_outputs)

    def transform(self, graphs):
        """tm.py:814-851: (int32 [graphs][clauses] = the clause is true at some node, class sums)."""
        return self._transform(graphs, False)

    def transform_nodewise(self, graphs):
        """tm.py:853-900: (int32 [graphs][clauses][largest graph] = the clause's truth per node, class sums)."""
        return self._transform(graphs, True)

    # ------------------------------------------------------------- state I/O

    def _download(self):
        C, B = self.number_of_clauses, self.number_of_state_bits
        self.ta_state = self.ta_state_gpu.cpu().numpy().view(np.uint32).reshape(C * self.number_of_ta_chunks * B)
        self.message_ta_state = [t.cpu().numpy().view(np.uint32) for t in self.message_ta_state_gpu]
        self.clause_weights = self.clause_weights_gpu.cpu().numpy()

    def ta_action(self, depth, clause, ta):
        """tm.py:126-142: is literal `ta` of `clause` included at layer `depth`?"""
        self._download()
        B = self.number_of_state_bits
        if depth == 0:
            bank = self.ta_state.reshape(self.number_of_clauses, self.number_of_ta_chunks, B)
        else:
            bank = self.message_ta_state[depth - 1].reshape(self.number_of_clauses, self.number_of_message_chunks, B)
        return (bank[clause, ta // 32, B - 1] & (1 << (ta % 32))) > 0

    def _read_bank(self, entry, depth):
        if depth == 0:
            bank, chunks, literals = self.ta_state_gpu, self.number_of_ta_chunks, self.number_of_literals
        else:
            bank = self.message_ta_state_gpu[depth - 1]
            chunks, literals = self.number_of_message_chunks, self.number_of_message_literals
        cfg = self._config(max(self._max_nodes_seen(), 1))
        out = torch.empty(self.number_of_clauses * literals, dtype=torch.int32, device=_device())
        _abi.call(entry, ctypes.byref(cfg), _ptr(bank), chunks, literals, _ptr(out), _stream())
        return out.cpu().numpy().view(np.uint32).reshape(self.number_of_clauses, literals)

    def _max_nodes_seen(self):
        return self._train_graphs.max_nodes if self._train_graphs is not None else 1

    def get_hyperliterals(self, depth):
        """tm.py:144-172: uint32 [clauses][literals of the layer], 1 where the automaton includes."""
        return self._read_bank("gtm_get_hyperliterals", depth)

    def get_ta_states(self, depth):
        """tm.py:174-205: uint32 [clauses][literals of the layer], the automata's integer states."""
        return self._read_bank("gtm_get_ta_states", depth)

    def get_clause_literals(self, symbol_hv):
        """tm.py:213-240: float [clauses][2 * symbols], how many of each symbol's hypervector
        bits the clause includes (second half: their negations)."""
        hv_clauses = self.get_hyperliterals(0)
        half = self.number_of_literals // 2
        n_symbols = symbol_hv.shape[0]
        expanded = np.zeros((half, n_symbols), dtype=np.uint8)
        for sym_id in range(n_symbols):
            expanded[symbol_hv[sym_id].ravel(), sym_id] = 1
        out = np.zeros((self.number_of_clauses, 2 * n_symbols))
        out[:, :n_symbols] = hv_clauses[:, :half] @ expanded
        out[:, n_symbols:] = hv_clauses[:, half:] @ expanded
        return out

    def get_messages(self, depth, edge_types):
        """tm.py:242-279: float [edge types][clauses][2 * clauses], how many of each sending
        clause's (rotated) hypervector bits a clause's message literals of layer `depth` include."""
        assert depth > 0, f"Expected depth > 0, got {depth}. Depth <= 0 means surface, use get_clause_literals()"
        hv_messages = self.get_hyperliterals(depth).astype(np.float32)
        half, C = self.number_of_message_literals // 2, self.number_of_clauses
        out = np.zeros((edge_types, C, 2 * C))
        for edge_type in range(edge_types):
            expanded = np.zeros((half, C))
            for sym_id in range(C):
                expanded[(self.hypervectors[sym_id].ravel() + edge_type) % self.message_size, sym_id] = 1
            out[edge_type, :, :C] = hv_messages[:, :half] @ expanded
            out[edge_type, :, C:] = hv_messages[:, half:] @ expanded
        return out

    def get_weights(self):
        """tm.py:207-211."""
        if np.array_equal(self.clause_weights, np.array([])):
            self.clause_weights = self.clause_weights_gpu.cpu().numpy()
        return self.clause_weights.reshape((self.number_of_outputs, self.number_of_clauses))

    def get_state(self):
        """tm.py:281-287: the 10-tuple, always read fresh from the device.  The
        tuple also carries the message banks as the attribute
        ``message_ta_state`` (the reference's tuple leaves them out), so that
        ``set_state(get_state())`` restores a model with message layers
        completely."""
        self._download()
        state = ModelState((
            self.ta_state, self.clause_weights, self.number_of_outputs, self.number_of_clauses,
            self.number_of_literals, self.depth, self.number_of_state_bits, self.number_of_ta_chunks,
            self.min_y, self.max_y,
        ))
        state.message_ta_state = list(self.message_ta_state)
        return state

    def set_state(self, state):
        """tm.py:289-310, made to leave a usable model: works on a model that
        has never been trained (every buffer is allocated here), restores the
        layer-0 bank and the weights from the tuple and the message banks from
        its ``message_ta_state`` attribute when it has one (tuples made by
        this class's ``get_state``).  A plain 10-tuple, as the reference makes
        them, holds no message banks: those keep their contents on an
        initialised model of the same shape and start from the initial state
        otherwise."""
        (ta_state, weights, outputs, clauses, literals, depth, state_bits, ta_chunks, min_y, max_y) = tuple(state)
        same_shape = self.initialized and (
            int(outputs), int(clauses), int(literals), int(depth), int(state_bits)
        ) == (
            getattr(self, "_allocated_outputs", -1), self.number_of_clauses, self.number_of_literals, self.depth,
            self.number_of_state_bits,
        )
        if int(depth) != self.depth and self.one_hot_encoding:
            raise _abi.GtmError("set_state cannot change the depth of a one-hot model; use load()")
        if not same_shape and self.one_hot_encoding and int(depth) > 1 and not self.initialized:
            raise _abi.GtmError(
                "a one-hot model takes its message size from the first data set's edge types; "
                "use load() to build it from a saved state"
            )
        ta_state = np.ascontiguousarray(ta_state, dtype=np.uint32).reshape(-1)
        weights = np.ascontiguousarray(weights, dtype=np.int32).reshape(-1)
        chunks = int((int(literals) - 1) // 32 + 1)
        bank_words = int(clauses) * chunks * int(state_bits)
        # the reference allocates depth x the layer-0 bank (tm.py:299) and copies the whole array:
        # only the first bank's worth is the layer-0 state
        if ta_state.size < bank_words or weights.size != int(outputs) * int(clauses) or int(ta_chunks) != chunks:
            raise _abi.GtmError("set_state: array sizes do not match the sizes in the tuple")
        banks = getattr(state, "message_ta_state", None)
        if not same_shape:
            if int(clauses) != self.number_of_clauses and int(depth) > 1:
                raise _abi.GtmError("set_state cannot change the number of clauses of a model with message layers "
                                    "(its hypervectors have one row per clause); use load()")
            self.number_of_outputs = int(outputs)
            self.number_of_clauses = int(clauses)
            self.number_of_clause_chunks = (self.number_of_clauses - 1) // 32 + 1
            self.number_of_literals = int(literals)
            if int(depth) != self.depth:
                self.s = tuple(self.s[i] if i < len(self.s) else self.s[-1] for i in range(int(depth)))
            self.depth = int(depth)
            self.number_of_state_bits = int(state_bits)
            self.number_of_ta_chunks = chunks
            self.number_of_features = self.number_of_literals // 2
            self.number_of_message_features = self.message_size
            self.number_of_message_literals = self.message_size * 2
            self.number_of_message_chunks = int((self.number_of_message_literals - 1) // 32 + 1)
            if self.max_included_literals is None:
                self.max_included_literals = self.number_of_literals
            if not hasattr(self, "max_number_of_graph_nodes"):
                self.max_number_of_graph_nodes = 0  # taken from the data set of every call
            self._allocate()
            self.initialized = True
            if banks is None and self.depth > 1:
                cfg = self._config(1)
                for t in self.message_ta_state_gpu:
                    _abi.call("gtm_prepare_message_ta_state", ctypes.byref(cfg), _ptr(t), _stream())
        self.min_y, self.max_y = min_y, max_y
        self.ta_state_gpu.copy_(_to_device(ta_state[:bank_words]))
        self.clause_weights_gpu.copy_(_to_device(weights))
        if banks is not None:
            if len(banks) != self.depth - 1:
                raise _abi.GtmError("set_state: %d message banks for depth %d" % (len(banks), self.depth))
            for t, host in zip(self.message_ta_state_gpu, banks):
                host = np.ascontiguousarray(host, dtype=np.uint32).reshape(-1)
                if host.size != t.numel():
                    raise _abi.GtmError("set_state: a message bank has %d words, expected %d" % (host.size, t.numel()))
                t.copy_(_to_device(host))
        self.graphs_signature_train = np.array([])
        self.graphs_signature_test = np.array([])
        self._train_graphs = self._test_graphs = None
        self.encoded_Y = np.array([])
        self._encoded_Y_gpu = None
        self.ta_state = np.array([])
        self.clause_weights = np.array([])

    def save(self, fname="", format=None):
        """tm.py:312-362: the reference's 24 keys plus the generator position.  The file is a NumPy
        archive of plain arrays (nothing in it is pickled, so reading it back runs nothing) unless
        ``format="pickle"`` asks for the reference's pickle of the same dict (tm.py:356-357), for
        files that the reference itself is to load.  ``load`` tells the two apart by their first
        bytes, whatever the file is called."""
        if format not in (None, "npz", "pickle"):
            raise _abi.GtmError("save: format=%r is neither 'npz' nor 'pickle'" % (format,))
        self._download()
        state_dict = {
            "ta_state": self.ta_state,
            "message_ta_state": self.message_ta_state,
            "clause_weights": self.clause_weights,
            "hypervectors": self.hypervectors,
            "number_of_outputs": self.number_of_outputs,
            "number_of_literals": self.number_of_literals,
            "number_of_message_literals": self.number_of_message_literals,
            "min_y": self.min_y,
            "max_y": self.max_y,
            "negative_clauses": self.negative_clauses,
            "max_number_of_graph_nodes": self.max_number_of_graph_nodes,
            "number_of_clauses": self.number_of_clauses,
            "T": self.T,
            "s": self.s,
            "q": self.q,
            "max_included_literals": self.max_included_literals,
            "boost_true_positive_feedback": self.boost_true_positive_feedback,
            "number_of_state_bits": self.number_of_state_bits,
            "depth": self.depth,
            "message_size": self.message_size,
            "message_bits": self.message_bits,
            "double_hashing": self.double_hashing,
            "one_hot_encoding": self.one_hot_encoding,
            # not in the reference: where the counter-based generator stands
            "rng_seed": self.seed,
            "rng_step": self.step,
        }
        if len(fname) > 0:
            print(f"Saving model to {fname}.")
            if format == "pickle":
                with open(fname, "wb") as f:
                    pickle.dump(state_dict, f)
            else:
                write_state_npz(state_dict, fname)
        return state_dict

    def load(self, state_dict={}, fname=""):
        """tm.py:364-412.  A file is read as the NumPy archive that ``save`` writes or, when it is a
        pickle (``save(format="pickle")``, or the reference's own ``save``), by an unpickler that only
        rebuilds arrays, scalars and plain containers and refuses every other global a pickle names."""
        if len(fname) == 0 and len(state_dict) == 0:
            print("Error: No file or state_dict provided. Pass either a file name or a state_dict.")
            return
        if len(fname) > 0:
            print(f"Loading model from {fname}.")
            with open(fname, "rb") as f:
                is_archive = f.read(2) == b"PK"  # a NumPy archive is a zip file
            state_dict = read_state_npz(fname) if is_archive else read_state_pickle(fname)
        # the constructor arguments travel with the state (tm.py:341-353 saves them; the reference's
        # load leaves them to the caller's constructor call): a model built with other arguments
        # must not run a loaded state with the wrong clause count, depth or automaton width
        for key in ("number_of_clauses", "T", "s", "q", "max_included_literals", "boost_true_positive_feedback",
                    "number_of_state_bits", "depth", "message_bits", "double_hashing", "one_hot_encoding"):
            if key in state_dict:
                setattr(self, key, state_dict[key])
        self.number_of_clause_chunks = (self.number_of_clauses - 1) // 32 + 1
        self.s = tuple(self.s) if isinstance(self.s, (tuple, list)) else (self.s,) * self.depth
        self.ta_state = state_dict["ta_state"]
        self.message_ta_state = state_dict["message_ta_state"]
        self.clause_weights = state_dict["clause_weights"]
        self.hypervectors = state_dict["hypervectors"]
        self.number_of_outputs = state_dict["number_of_outputs"]
        self.number_of_literals = state_dict["number_of_literals"]
        self.number_of_message_literals = state_dict["number_of_message_literals"]
        self.min_y = state_dict["min_y"]
        self.max_y = state_dict["max_y"]
        self.negative_clauses = state_dict["negative_clauses"]
        self.max_number_of_graph_nodes = state_dict["max_number_of_graph_nodes"]
        self.message_size = state_dict["message_size"]
        self.seed = int(state_dict.get("rng_seed", self.seed))
        self.step = int(state_dict.get("rng_step", 0))

        self.number_of_features = self.number_of_literals // 2
        self.number_of_ta_chunks = int((self.number_of_literals - 1) // 32 + 1)
        self.number_of_message_features = self.number_of_message_literals // 2
        self.number_of_message_chunks = int((self.number_of_message_literals - 1) // 32 + 1)
        if self.max_included_literals is None:
            self.max_included_literals = self.number_of_literals

        C, B = self.number_of_clauses, self.number_of_state_bits
        expected = [("ta_state", self.ta_state, C * self.number_of_ta_chunks * B),
                    ("clause_weights", self.clause_weights, self.number_of_outputs * C),
                    ("hypervectors", self.hypervectors, C * self.message_bits)]
        if len(self.message_ta_state) != self.depth - 1:
            raise _abi.GtmError("state has %d message banks for depth %d" % (len(self.message_ta_state), self.depth))
        expected += [("message_ta_state[%d]" % i, b, C * self.number_of_message_chunks * B)
                     for i, b in enumerate(self.message_ta_state)]
        for name, array, size in expected:
            if np.asarray(array).size != size:
                raise _abi.GtmError("state's %s has %d elements, expected %d" % (name, np.asarray(array).size, size))
        self.hypervectors = np.ascontiguousarray(self.hypervectors, dtype=np.uint32).reshape(C, self.message_bits)
        self._allocate()
        self.ta_state_gpu.copy_(_to_device(np.asarray(self.ta_state, dtype=np.uint32)))
        for t, host in zip(self.message_ta_state_gpu, self.message_ta_state):
            t.copy_(_to_device(np.asarray(host, dtype=np.uint32)))
        self.clause_weights_gpu.copy_(_to_device(np.asarray(self.clause_weights, dtype=np.int32)))
        self._train_graphs = self._test_graphs = None
        self.encoded_Y = np.array([])
        self._encoded_Y_gpu = None
        self.graphs_signature_train = np.array([])
        self.graphs_signature_test = np.array([])
        self.initialized = True


class MultiClassGraphTsetlinMachine(CommonTsetlinMachine):
    """tm.py:903-959."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.negative_clauses = 1

    def fit(self, graphs, Y, epochs=100, incremental=False, examples=None):
        Y = np.asarray(Y)
        self.number_of_outputs = self._outputs_for(int(np.max(Y) + 1))
        self.max_y = None
        self.min_y = None
        encoded_Y = np.empty((Y.shape[0], self.number_of_outputs), dtype=np.int32)
        for i in range(self.number_of_outputs):
            encoded_Y[:, i] = np.where(Y == i, self.T, -self.T)
        self._fit(graphs, encoded_Y, epochs=epochs, incremental=incremental, examples=examples)

    def score(self, graphs):
        return self._score(graphs)

    def predict(self, graphs):
        return np.argmax(self.score(graphs), axis=1)


class MultiOutputGraphTsetlinMachine(CommonTsetlinMachine):
    """tm.py:961-1017."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.negative_clauses = 1

    def fit(self, graphs, Y, epochs=100, incremental=False):
        Y = np.asarray(Y)
        if self._outputs_for(Y.shape[1]) != Y.shape[1]:
            raise _abi.GtmError("this model has %d outputs; Y has %d columns" % (self._allocated_outputs, Y.shape[1]))
        self.number_of_outputs = Y.shape[1]
        self.max_y = None
        self.min_y = None
        encoded_Y = np.where(Y == 1, self.T, -self.T).astype(np.int32)
        self._fit(graphs, encoded_Y, epochs=epochs, incremental=incremental)

    def score(self, graphs):
        return self._score(graphs)

    def predict(self, graphs):
        return (self.score(graphs) >= 0).astype(np.uint32)


class GraphTsetlinMachine(CommonTsetlinMachine):
    """tm.py:1019-1072."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.negative_clauses = 1

    def fit(self, graphs, Y, epochs=100, incremental=False):
        self.number_of_outputs = 1
        self.max_y = None
        self.min_y = None
        encoded_Y = np.where(np.asarray(Y) == 1, self.T, -self.T).astype(np.int32).reshape(-1, 1)
        self._fit(graphs, encoded_Y, epochs=epochs, incremental=incremental)

    def score(self, graphs):
        return self._score(graphs)[:, 0]

    def predict(self, graphs):
        return self.score(graphs) >= 0
