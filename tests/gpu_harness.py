"""Thin wrappers that call the C-ABI entry points one operator at a time on
torch-owned device buffers and bring results back as NumPy arrays in the
oracle's shapes.  Imported only by GPU tests."""

import ctypes

import numpy as np
import torch

from graphtsetlinmachine_amd import _abi
from graphtsetlinmachine_amd.tm import _DeviceGraphs, _ptr, _stream, _to_device


def abi_config(cfg, depth, s, seed):
    s = tuple(s) if isinstance(s, (tuple, list)) else (s,) * depth
    return _abi.make_config(
        classes=cfg.classes, clauses=cfg.clauses, literals=cfg.literals, state_bits=cfg.state_bits,
        boost_true_positive_feedback=cfg.boost_true_positive_feedback, threshold=cfg.threshold, q=cfg.q,
        max_included_literals=cfg.max_included_literals, negative_clauses=cfg.negative_clauses,
        max_nodes=cfg.max_nodes, message_size=cfg.message_size, message_bits=cfg.message_bits, depth=depth,
        s=s, seed=seed,
    )


def dev_u32(shape_or_array):
    if isinstance(shape_or_array, np.ndarray):
        return _to_device(shape_or_array)
    n = int(np.prod(shape_or_array))
    return torch.full((max(n, 1),), 0x5A5A5A5A, dtype=torch.int32, device="cuda")


def host(t, dtype, shape):
    return t.cpu().numpy().view(dtype)[: int(np.prod(shape))].reshape(shape).copy()


class Device:
    """One oracle Model + one Graphs mirrored on the GPU."""

    def __init__(self, model, graphs):
        self.model = model
        self.cfg = model.cfg
        self.graphs = graphs
        self.dg = _DeviceGraphs(graphs)
        self.acfg = abi_config(model.cfg, model.depth, model.s, model.seed)
        self.ta = _to_device(model.ta_state)
        self.banks = [_to_device(b) for b in model.message_ta_state]
        self.weights = _to_device(model.clause_weights)
        self.hv = _to_device(model.hypervectors)
        c = self.cfg
        self.inc = dev_u32((max(c.la_chunks, c.message_chunks), c.clauses))

    def state(self):
        st = _abi.State()
        st.ta_state = _ptr(self.ta)
        for i, b in enumerate(self.banks):
            st.message_ta_state[i] = b.data_ptr()
        st.clause_weights = _ptr(self.weights)
        st.hypervectors = _ptr(self.hv)
        return st

    # --- operators -------------------------------------------------------
    def calculate_messages(self, first, n):
        c = self.cfg
        out = dev_u32((n, c.clauses, c.node_chunks))
        n_incl = dev_u32((c.clauses,))
        _abi.call("gtm_calculate_messages", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), first, n,
                  _ptr(self.ta), _ptr(self.inc), _ptr(out), _ptr(n_incl), _stream())
        return out, n_incl

    def exchange_messages(self, first, n, bitmap):
        c = self.cfg
        cx = dev_u32((n, c.max_nodes, c.message_chunks))
        _abi.call("gtm_exchange_messages", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), first, n,
                  _ptr(self.hv), _ptr(bitmap), _ptr(cx), _stream())
        return cx

    def calculate_messages_conditional(self, first, n, layer, cond, n_incl, cx):
        c = self.cfg
        out = dev_u32((n, c.clauses, c.node_chunks))
        _abi.call("gtm_calculate_messages_conditional", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), first, n,
                  _ptr(self.banks[layer]), _ptr(self.inc), _ptr(cond), _ptr(out), _ptr(n_incl), _ptr(cx), _stream())
        return out

    def evaluate(self, first, n, bitmap):
        out = dev_u32((n, self.cfg.classes))
        _abi.call("gtm_evaluate", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), first, n, _ptr(bitmap),
                  _ptr(self.weights), _ptr(out), _stream())
        return out

    def select_clause_node(self, example, step, bitmap):
        out = dev_u32((self.cfg.clauses,))
        _abi.call("gtm_select_clause_node", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), example, step,
                  _ptr(bitmap), _ptr(out), _stream())
        return out

    def select_clause_updates(self, step, class_sum, encoded_Y, example, clause_node):
        out = dev_u32((self.cfg.classes, self.cfg.clauses))
        y = _to_device(np.ascontiguousarray(encoded_Y, dtype=np.int32))
        _abi.call("gtm_select_clause_updates", ctypes.byref(self.acfg), step, _ptr(self.weights), _ptr(class_sum),
                  _ptr(y), example, _ptr(clause_node), _ptr(out), _stream())
        torch.cuda.synchronize()
        return out

    def update(self, example, step, clause_node, n_incl, updates):
        _abi.call("gtm_update", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), example, step, _ptr(self.ta),
                  _ptr(clause_node), _ptr(n_incl), _ptr(updates), _stream())

    def update_message(self, step, bank, clause_node, n_incl, cx, updates):
        _abi.call("gtm_update_message", ctypes.byref(self.acfg), step, bank, _ptr(self.banks[bank - 1]),
                  _ptr(clause_node), _ptr(n_incl), _ptr(cx), _ptr(updates), _stream())

    # --- driver loops ----------------------------------------------------
    def properties(self):
        """(some negated literal is not its positive one's complement, some graph has no nodes)"""
        found = torch.full((2,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
        _abi.call("gtm_graphs_properties", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), _ptr(found), _stream())
        return tuple(int(v) for v in found.cpu().numpy())

    def declare_complementary(self):
        """Set GTM_GRAPHS_COMPLEMENTARY if the data set passes the library's check."""
        ok = self.properties() == (0, 0)
        self.dg.desc.flags = _abi.GTM_GRAPHS_COMPLEMENTARY if ok else 0
        return ok

    def build_tiles(self):
        nbytes = _abi.lib.gtm_tiles_bytes(ctypes.byref(self.acfg), ctypes.byref(self.dg.desc))
        if nbytes == 0:
            return False
        self.tiles = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda")
        _abi.call("gtm_build_tiles", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), _ptr(self.tiles), _stream())
        self.dg.desc.tiles = self.tiles.data_ptr()
        return True

    def score(self, first, n, batch):
        need = _abi.lib.gtm_score_workspace_bytes(ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), batch)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        out = dev_u32((n, self.cfg.classes))
        st = self.state()
        _abi.call("gtm_score", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), ctypes.byref(st), first, n, batch,
                  _ptr(ws), ws.numel(), _ptr(out), _stream())
        return host(out, np.int32, (n, self.cfg.classes))

    def fit(self, encoded_Y, first, n, first_step, tiles=False):
        if tiles:
            assert self.build_tiles()
        need = _abi.lib.gtm_fit_workspace_bytes(ctypes.byref(self.acfg), ctypes.byref(self.dg.desc))
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        y = _to_device(np.ascontiguousarray(encoded_Y, dtype=np.int32))
        st = self.state()
        _abi.call("gtm_fit", ctypes.byref(self.acfg), ctypes.byref(self.dg.desc), ctypes.byref(st), _ptr(y), first, n,
                  first_step, _ptr(ws), ws.numel(), _stream())
        torch.cuda.synchronize()

    def download(self):
        c = self.cfg
        ta = host(self.ta, np.uint32, (c.clauses, c.la_chunks, c.state_bits))
        banks = [host(b, np.uint32, (c.clauses, c.message_chunks, c.state_bits)) for b in self.banks]
        w = host(self.weights, np.int32, (c.classes, c.clauses))
        return ta, banks, w
