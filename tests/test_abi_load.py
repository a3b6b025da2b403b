"""The C-ABI library loads, exports every symbol that include/gtm_abi.h
declares, and the ctypes structures have the layout the C compiler gives the
header's structs.  No compute calls: this runs without a GPU."""

import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gtm_abi.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gtm_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from graphtsetlinmachine_amd import _abi

    names = declared_functions()
    assert len(names) >= 16
    for name in names:
        assert hasattr(_abi.lib, name), "libgtm_hip.so lacks %s" % name
        assert name in _abi.PROTOTYPES, "no ctypes prototype for %s" % name
    assert sorted(_abi.PROTOTYPES) == names
    assert _abi.lib.gtm_abi_version() == _abi.GTM_ABI_VERSION


def test_invalid_config_is_rejected_without_touching_the_gpu():
    from graphtsetlinmachine_amd import _abi

    cfg = _abi.make_config(classes=2, clauses=0, literals=8, state_bits=8, boost_true_positive_feedback=1,
                           threshold=10, q=1.0, max_included_literals=8, negative_clauses=1, max_nodes=1,
                           message_size=8, message_bits=2, depth=1, s=(1.0,), seed=1)
    with pytest.raises(_abi.GtmError, match="clauses=0"):
        _abi.call("gtm_prepare_message_ta_state", ctypes.byref(cfg), None, None)
    assert _abi.lib.gtm_score_workspace_bytes(ctypes.byref(cfg), None, 4) == 0


def test_switches_are_read_at_load_and_changed_only_through_the_library(monkeypatch):
    """The library looks at the environment once, when it is loaded: a variable set afterwards changes
    nothing until gtm_tuning_reload; gtm_tuning_set sets and unsets one switch; unknown names and
    over-long values are refused."""
    from graphtsetlinmachine_amd import _abi

    name = "GTM_WIDE_SPLITS"
    before = _abi.tuning(name)
    try:
        monkeypatch.setenv(name, "7")
        assert _abi.tuning(name) == before          # the environment is not read per call
        _abi.call("gtm_tuning_reload")
        assert _abi.tuning(name) == "7"
        _abi.call("gtm_tuning_set", name.encode(), b"3")
        assert _abi.tuning(name) == "3"
        _abi.call("gtm_tuning_set", name.encode(), None)
        assert _abi.tuning(name) is None
        with pytest.raises(_abi.GtmError, match="not a switch"):
            _abi.call("gtm_tuning_set", b"GTM_NO_SUCH_SWITCH", b"1")
        with pytest.raises(_abi.GtmError, match="longer than"):
            _abi.call("gtm_tuning_set", name.encode(), b"1" * 64)
        assert _abi.tuning("GTM_NO_SUCH_SWITCH") is None
    finally:
        monkeypatch.delenv(name, raising=False)
        _abi.call("gtm_tuning_reload")
    assert _abi.tuning(name) is None or _abi.tuning(name) == os.environ.get(name)


def test_ctypes_structs_match_the_header(tmp_path):
    from graphtsetlinmachine_amd import _abi

    fields = {
        "gtm_config": [f[0] for f in _abi.Config._fields_],
        "gtm_graphs": [f[0] for f in _abi.GraphsDesc._fields_],
        "gtm_state": [f[0] for f in _abi.State._fields_],
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "gtm_abi.h"', "int main(void){"]
    for struct, names in fields.items():
        lines.append('printf("%s %%zu\\n", sizeof(%s));' % (struct, struct))
        for n in names:
            lines.append('printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (struct, n, struct, n))
    lines.append("return 0;}")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for struct, cls in (("gtm_config", _abi.Config), ("gtm_graphs", _abi.GraphsDesc), ("gtm_state", _abi.State)):
        assert int(out[struct]) == ctypes.sizeof(cls)
        for n in fields[struct]:
            assert int(out["%s.%s" % (struct, n)]) == getattr(cls, n).offset, "%s.%s" % (struct, n)


def test_product_package_does_not_import_the_oracle():
    """The shipped path must not route through the CPU oracle."""
    pkg = os.path.join(ROOT, "graphtsetlinmachine_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def _desc(n_graphs, max_nodes, n_types=1, edges_per_graph=0, tiles=0):
    from graphtsetlinmachine_amd import _abi

    d = _abi.GraphsDesc()
    d.number_of_graphs = n_graphs
    d.number_of_node_types = n_types
    d.max_number_of_graph_nodes = max_nodes
    d.total_nodes = n_graphs * max_nodes
    d.total_edges = n_graphs * edges_per_graph
    d.tiles = tiles
    return d


def test_buffer_sizes_are_computed_in_64_bits_at_and_beyond_the_largest_configuration():
    """The colour configuration at its full data-set size (50,000 graphs of 841 nodes, 2,048 literals, 8,000
    clauses, depth 3: X alone is 10.8 GB) and ten times that: every size the host hands out is the
    product it should be, far beyond 2^32 - no offset of the driver loops is formed in 32 bits.  (Host
    arithmetic only: nothing is launched.)"""
    from graphtsetlinmachine_amd import _abi

    cfg = _abi.make_config(classes=10, clauses=8000, literals=2048, state_bits=8, boost_true_positive_feedback=1,
                           threshold=10000, q=1.0, max_included_literals=2048, negative_clauses=1, max_nodes=841,
                           message_size=1024, message_bits=2, depth=3, s=(15.0,) * 3, seed=1)
    for n_graphs in (50000, 500000):
        d = _desc(n_graphs, 841, edges_per_graph=3248)
        # message rows (1,026) rule the tile: one 841-node graph (27 -> 28 words per row) per tile
        rows, tw = 2048 + 1 + 1, 28
        want = n_graphs * rows * tw * 4 + rows * 8 + 2048 * 4
        got = _abi.lib.gtm_tiles_bytes(ctypes.byref(cfg), ctypes.byref(d))
        assert got == want and got > 2**33
        # the dense path's workspace grows with the batch: [batch][CLAUSES][NODE_CHUNKS] bitmaps twice and
        # [batch][max_nodes][MESSAGE_CHUNKS] packed messages
        small = _abi.lib.gtm_score_workspace_bytes(ctypes.byref(cfg), ctypes.byref(d), 1)
        big = _abi.lib.gtm_score_workspace_bytes(ctypes.byref(cfg), ctypes.byref(d), 1 << 16)
        per_graph = 2 * 8000 * 27 * 4 + 841 * 64 * 4
        assert big - small == ((1 << 16) - 1) * per_graph and big > 2**36
    # the 361-node configuration with 6 million graphs: X = 69 GB, tiles of all rows 10 graphs each
    conv = _abi.make_config(classes=10, clauses=2500, literals=256, state_bits=8, boost_true_positive_feedback=1,
                            threshold=3125, q=1.0, max_included_literals=256, negative_clauses=1, max_nodes=361,
                            message_size=256, message_bits=2, depth=1, s=(10.0,), seed=1)
    d = _desc(6_000_000, 361)
    assert _abi.lib.gtm_tiles_bytes(ctypes.byref(conv), ctypes.byref(d)) == 600_000 * 258 * 128 * 4 + 258 * 8 + 256 * 4
    # and declared complementary: 21 graphs per tile of 256-word rows, plus 16 bytes per node slot
    d.flags = _abi.GTM_GRAPHS_COMPLEMENTARY
    n_tiles = (6_000_000 + 20) // 21
    rows_part = n_tiles * 258 * 256 * 4 + 258 * 8 + 256 * 4
    assert rows_part % 16 == 0
    assert _abi.lib.gtm_tiles_bytes(ctypes.byref(conv), ctypes.byref(d)) == rows_part + n_tiles * 256 * 32 * 16
