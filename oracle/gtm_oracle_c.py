"""ctypes front end of oracle/gtm_oracle.c, the C restatement of the inference path.

TEST INFRASTRUCTURE ONLY (tests, the smoke check, bench.py's CPU-baseline leg).
``build()`` compiles the C file with gcc into oracle/libgtm_oracle_c.so; ``score``
builds it on first use when the library is missing and gcc is there.
"""

import ctypes as C
import os
import shutil
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(HERE, "gtm_oracle.c")
LIBRARY = os.path.join(HERE, "libgtm_oracle_c.so")

_lib = None


class _Config(C.Structure):
    _fields_ = [(name, C.c_int32) for name in
                ("classes", "clauses", "literals", "state_bits", "max_nodes", "message_size", "message_bits", "depth")]


class _Graphs(C.Structure):
    _fields_ = [(name, C.c_void_p) for name in
                ("X", "node_type", "number_of_graph_node_edges", "edge", "node_index", "edge_index",
                 "number_of_graph_nodes")] + [("number_of_node_types", C.c_int32)]


def build(verbose=False):
    cmd = ["gcc", "-O3", "-fopenmp", "-shared", "-fPIC", "-o", LIBRARY, SOURCE]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIBRARY


def available():
    return os.path.exists(LIBRARY) or shutil.which("gcc") is not None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY) or os.path.getmtime(LIBRARY) < os.path.getmtime(SOURCE):
            build()
        _lib = C.CDLL(LIBRARY)
        _lib.gtmc_score.restype = C.c_int
        _lib.gtmc_fit.restype = C.c_int
        _lib.gtmc_threads_available.restype = C.c_int
    return _lib


class _Training(C.Structure):
    _fields_ = [("threshold", C.c_int32), ("boost_true_positive_feedback", C.c_int32),
                ("max_included_literals", C.c_int32), ("negative_clauses", C.c_int32),
                ("q_threshold", C.c_uint64), ("seed", C.c_uint64), ("feedback_threshold", C.c_uint32 * 8)]


def threads_available():
    return int(_load().gtmc_threads_available())


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def score(model, graphs, indices=None, threads=1):
    """Class sums int32 ``[len(indices)][classes]`` of an oracle ``Model`` (oracle/gtm_oracle.py)
    on ``graphs``: the same call as ``gtm_oracle.score``."""
    lib = _load()
    cfg = model.cfg
    ids = np.arange(graphs.number_of_graphs) if indices is None else np.asarray(list(indices))
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    keep = [_u32(graphs.X), _u32(graphs.node_type), _u32(graphs.number_of_graph_node_edges),
            _u32(np.asarray(graphs.edge).reshape(-1)), _u32(graphs.node_index), _u32(graphs.edge_index),
            _u32(graphs.number_of_graph_nodes)]
    if keep[3].size == 0:
        keep[3] = np.zeros(2, dtype=np.uint32)
    g = _Graphs(*[a.ctypes.data for a in keep], int(graphs.number_of_node_types()))
    c = _Config(cfg.classes, cfg.clauses, cfg.literals, cfg.state_bits, cfg.max_nodes, cfg.message_size,
                cfg.message_bits, model.depth)
    ta = _u32(model.ta_state)
    banks = [_u32(b) for b in model.message_ta_state]
    bank_ptrs = (C.c_void_p * max(1, len(banks)))(*[b.ctypes.data for b in banks])
    weights = np.ascontiguousarray(model.clause_weights, dtype=np.int32)
    hv = _u32(model.hypervectors)
    out = np.empty((ids.size, cfg.classes), dtype=np.int32)
    rc = lib.gtmc_score(C.byref(c), C.byref(g), C.c_void_p(ta.ctypes.data), bank_ptrs,
                        C.c_void_p(weights.ctypes.data), C.c_void_p(hv.ctypes.data), C.c_void_p(ids.ctypes.data),
                        C.c_int32(ids.size), C.c_int32(threads), C.c_void_p(out.ctypes.data))
    if rc != 0:
        raise MemoryError("gtmc_score could not allocate its scratch buffers")
    return out


def fit(model, graphs, encoded_Y, epochs=1, indices=None, threads=1):
    """``gtm_oracle.fit`` in C: trains the oracle ``Model`` in place (banks, weights, step)."""
    from oracle import gtm_oracle as o

    lib = _load()
    cfg = model.cfg
    if model.depth > 8:
        raise ValueError("at most 8 banks")
    ids = np.arange(graphs.number_of_graphs) if indices is None else np.asarray(list(indices))
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    keep = [_u32(graphs.X), _u32(graphs.node_type), _u32(graphs.number_of_graph_node_edges),
            _u32(np.asarray(graphs.edge).reshape(-1)), _u32(graphs.node_index), _u32(graphs.edge_index),
            _u32(graphs.number_of_graph_nodes)]
    if keep[3].size == 0:
        keep[3] = np.zeros(2, dtype=np.uint32)
    g = _Graphs(*[a.ctypes.data for a in keep], int(graphs.number_of_node_types()))
    c = _Config(cfg.classes, cfg.clauses, cfg.literals, cfg.state_bits, cfg.max_nodes, cfg.message_size,
                cfg.message_bits, model.depth)
    t = _Training(cfg.threshold, cfg.boost_true_positive_feedback, cfg.max_included_literals, cfg.negative_clauses,
                  o.q_threshold(cfg.q, cfg.classes), int(model.seed) & 0xFFFFFFFFFFFFFFFF,
                  (C.c_uint32 * 8)(*[o.feedback_threshold(s) for s in np.atleast_1d(model.s)]))
    model.ta_state = _u32(model.ta_state)
    model.message_ta_state = [_u32(b) for b in model.message_ta_state]
    model.clause_weights = np.ascontiguousarray(model.clause_weights, dtype=np.int32)
    bank_ptrs = (C.c_void_p * max(1, len(model.message_ta_state)))(*[b.ctypes.data for b in model.message_ta_state])
    hv = _u32(model.hypervectors)
    y = np.ascontiguousarray(encoded_Y, dtype=np.int32)
    for _ in range(epochs):
        rc = lib.gtmc_fit(C.byref(c), C.byref(t), C.byref(g), C.c_void_p(model.ta_state.ctypes.data), bank_ptrs,
                          C.c_void_p(model.clause_weights.ctypes.data), C.c_void_p(hv.ctypes.data),
                          C.c_void_p(y.ctypes.data), C.c_void_p(ids.ctypes.data), C.c_int32(ids.size),
                          C.c_uint64(int(model.step)), C.c_int32(threads))
        if rc != 0:
            raise MemoryError("gtmc_fit could not allocate its scratch buffers")
        model.step += int(ids.size)
