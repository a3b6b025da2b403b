"""ctypes binding of libgtm_hip.so (the C ABI in include/gtm_abi.h).

There is no CPU fallback: if the library has not been built, importing this
module raises with the build command.
"""

import ctypes as C
import os

GTM_MAX_DEPTH = 8
GTM_ABI_VERSION = 3
GTM_GRAPHS_COMPLEMENTARY = 1

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libgtm_hip.so")


class GtmError(RuntimeError):
    pass


class Config(C.Structure):
    _fields_ = [
        ("classes", C.c_int32),
        ("clauses", C.c_int32),
        ("literals", C.c_int32),
        ("state_bits", C.c_int32),
        ("boost_true_positive_feedback", C.c_int32),
        ("threshold", C.c_int32),
        ("max_included_literals", C.c_int32),
        ("negative_clauses", C.c_int32),
        ("max_nodes", C.c_int32),
        ("message_size", C.c_int32),
        ("message_bits", C.c_int32),
        ("depth", C.c_int32),
        ("q", C.c_double),
        ("s", C.c_double * GTM_MAX_DEPTH),
        ("seed", C.c_uint64),
    ]


class GraphsDesc(C.Structure):
    _fields_ = [
        ("X", C.c_void_p),
        ("node_type", C.c_void_p),
        ("number_of_graph_node_edges", C.c_void_p),
        ("edge", C.c_void_p),
        ("node_index", C.c_void_p),
        ("edge_index", C.c_void_p),
        ("number_of_graph_nodes", C.c_void_p),
        ("number_of_graphs", C.c_int32),
        ("number_of_node_types", C.c_int32),
        ("max_number_of_graph_nodes", C.c_int32),
        ("flags", C.c_int32),
        ("total_nodes", C.c_int64),
        ("total_edges", C.c_int64),
        ("tiles", C.c_void_p),
    ]


class State(C.Structure):
    _fields_ = [
        ("ta_state", C.c_void_p),
        ("message_ta_state", C.c_void_p * (GTM_MAX_DEPTH - 1)),
        ("clause_weights", C.c_void_p),
        ("hypervectors", C.c_void_p),
    ]


_P = C.c_void_p
_CFG = C.POINTER(Config)
_GR = C.POINTER(GraphsDesc)
_ST = C.POINTER(State)
_I = C.c_int32
_U64 = C.c_uint64
_SZ = C.c_size_t

# name -> (restype, argtypes); mirrors include/gtm_abi.h one to one
PROTOTYPES = {
    "gtm_abi_version": (C.c_int, []),
    "gtm_last_error": (C.c_char_p, []),
    "gtm_prepare": (C.c_int, [_CFG, _U64, _P, _P, _P]),
    "gtm_prepare_message_ta_state": (C.c_int, [_CFG, _P, _P]),
    "gtm_calculate_messages": (C.c_int, [_CFG, _GR, _I, _I, _P, _P, _P, _P, _P]),
    "gtm_exchange_messages": (C.c_int, [_CFG, _GR, _I, _I, _P, _P, _P, _P]),
    "gtm_calculate_messages_conditional": (C.c_int, [_CFG, _GR, _I, _I, _P, _P, _P, _P, _P, _P, _P]),
    "gtm_evaluate": (C.c_int, [_CFG, _GR, _I, _I, _P, _P, _P, _P]),
    "gtm_select_clause_node": (C.c_int, [_CFG, _GR, _I, _U64, _P, _P, _P]),
    "gtm_select_clause_updates": (C.c_int, [_CFG, _U64, _P, _P, _P, _I, _P, _P, _P]),
    "gtm_update": (C.c_int, [_CFG, _GR, _I, _U64, _P, _P, _P, _P, _P]),
    "gtm_update_message": (C.c_int, [_CFG, _U64, _I, _P, _P, _P, _P, _P, _P]),
    "gtm_get_ta_states": (C.c_int, [_CFG, _P, _I, _I, _P, _P]),
    "gtm_get_hyperliterals": (C.c_int, [_CFG, _P, _I, _I, _P, _P]),
    "gtm_transform_workspace_bytes": (_SZ, [_CFG, _GR, _I]),
    "gtm_transform": (C.c_int, [_CFG, _GR, _ST, _I, _I, _I, _P, _SZ, _P, _P, _I, _P, _P]),
    "gtm_tuning_set": (C.c_int, [C.c_char_p, C.c_char_p]),
    "gtm_tuning_get": (C.c_char_p, [C.c_char_p]),
    "gtm_tuning_reload": (C.c_int, []),
    "gtm_profile_enable": (C.c_int, [C.c_int]),
    "gtm_profile_read": (C.c_int, [C.POINTER(C.c_char_p), C.POINTER(C.c_int32), C.POINTER(C.c_double)]),
    "gtm_profile_read_kernel": (C.c_int, [C.c_int32, C.POINTER(C.c_char_p), C.POINTER(C.c_int32), C.POINTER(C.c_double)]),
    "gtm_graphs_properties": (C.c_int, [_CFG, _GR, _P, _P]),
    "gtm_tiles_bytes": (_SZ, [_CFG, _GR]),
    "gtm_build_tiles": (C.c_int, [_CFG, _GR, _P, _P]),
    "gtm_score_workspace_bytes": (_SZ, [_CFG, _GR, _I]),
    "gtm_score": (C.c_int, [_CFG, _GR, _ST, _I, _I, _I, _P, _SZ, _P, _P]),
    "gtm_score_static_scratch_bytes": (_SZ, []),
    "gtm_score_static": (C.c_int, [_CFG, _GR, _ST, _I, _I, _I, _P, _P]),
    "gtm_fit_workspace_bytes": (_SZ, [_CFG, _GR]),
    "gtm_fit": (C.c_int, [_CFG, _GR, _ST, _P, _I, _I, _U64, _P, _SZ, _P]),
}

_STATUS_RETURNING = {name for name, (res, _) in PROTOTYPES.items() if res is C.c_int and name != "gtm_abi_version"}


def _load():
    if not os.path.exists(LIBRARY_PATH):
        raise GtmError(
            "%s is missing: the HIP library has not been built. Run "
            "`python -c 'import __graft_entry__ as g; g.build()'` at the repository root "
            "(or graphtsetlinmachine_amd/build.py)." % LIBRARY_PATH
        )
    # torch brings its own HIP runtime; loading it first makes this library bind to the same
    # one (two runtimes in a process do not see each other's device state)
    import torch  # noqa: F401

    lib = C.CDLL(LIBRARY_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.gtm_abi_version() != GTM_ABI_VERSION:
        raise GtmError("libgtm_hip.so has ABI version %d, expected %d" % (lib.gtm_abi_version(), GTM_ABI_VERSION))
    return lib


lib = _load()


def call(name, *args):
    """Call a status-returning entry point; raise GtmError with the library's
    message on failure."""
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise GtmError("%s failed (%d): %s" % (name, rc, lib.gtm_last_error().decode("utf-8", "replace")))


def tuning(name):
    """Value of one of the library's GTM_* switches as the library holds it (None = not set)."""
    v = lib.gtm_tuning_get(name.encode())
    return None if v is None else v.decode()


def make_config(
    classes, clauses, literals, state_bits, boost_true_positive_feedback, threshold, q, max_included_literals,
    negative_clauses, max_nodes, message_size, message_bits, depth, s, seed,
):
    if depth > GTM_MAX_DEPTH:
        raise GtmError("depth %d exceeds the supported maximum of %d" % (depth, GTM_MAX_DEPTH))
    cfg = Config()
    cfg.classes = classes
    cfg.clauses = clauses
    cfg.literals = literals
    cfg.state_bits = state_bits
    cfg.boost_true_positive_feedback = boost_true_positive_feedback
    cfg.threshold = threshold
    cfg.q = float(q)
    cfg.max_included_literals = max_included_literals
    cfg.negative_clauses = negative_clauses
    cfg.max_nodes = max_nodes
    cfg.message_size = message_size
    cfg.message_bits = message_bits
    cfg.depth = depth
    for i in range(GTM_MAX_DEPTH):
        cfg.s[i] = float(s[i]) if i < len(s) else 1.0
    cfg.seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    return cfg
