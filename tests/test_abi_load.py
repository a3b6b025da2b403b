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
