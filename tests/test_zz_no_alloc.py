"""gtm_score_static - the entry point that allocates nothing - against gtm_score
(which takes the caller's workspace), through the C ABI, bit for bit: two calls
in a row, the second on a smaller input, so that what the first call left in
the library's static scratch array is there when the second runs."""

import ctypes

import numpy as np
import pytest
import torch

from graphtsetlinmachine_amd import _abi
from graphtsetlinmachine_amd.tm import _ptr, _stream
from oracle import gtm_oracle as o
from tests import helpers

pytestmark = pytest.mark.gpu


def score_static(dev, first, n, batch):
    out = torch.full((max(n * dev.cfg.classes, 1),), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    st = dev.state()
    _abi.call("gtm_score_static", ctypes.byref(dev.acfg), ctypes.byref(dev.dg.desc), ctypes.byref(st), first, n, batch,
              _ptr(out), _stream())
    return out.cpu().numpy()[: n * dev.cfg.classes].reshape(n, dev.cfg.classes)


def device(seed, depth, n_graphs, max_nodes, clauses, classes, tiles, **graph_args):
    from tests.gpu_harness import Device

    graphs = helpers.random_graphs(seed, n_graphs=n_graphs, max_nodes=max_nodes, min_nodes=max(1, max_nodes // 2),
                                   hv_size=64, edge_types=("l", "r"), **graph_args)
    cfg = helpers.oracle_config(graphs, classes=classes, clauses=clauses, depth=depth, message_size=64, T=40)
    model = helpers.random_model(seed, cfg, depth, s=2.0, include_density=0.03)
    dev = Device(model, graphs)
    if tiles:
        assert dev.build_tiles()
    return dev, model, graphs


@pytest.mark.parametrize("depth, tiles", [(1, True), (2, True), (2, False)])
def test_two_calls_in_a_row_the_second_smaller_equal_gtm_score(depth, tiles):
    big, big_model, big_graphs = device(300 + depth, depth, n_graphs=60, max_nodes=90, clauses=300, classes=4, tiles=tiles)
    small, small_model, small_graphs = device(400 + depth, depth, n_graphs=9, max_nodes=20, clauses=40, classes=3,
                                              tiles=tiles)
    assert _abi.lib.gtm_score_static_scratch_bytes() == 16 << 20
    # first call: the larger model and data set, a batch that uses a good part of the scratch
    want_big = big.score(0, 60, 16)
    got_big = score_static(big, 0, 60, 16)
    assert np.array_equal(got_big, want_big)
    assert np.array_equal(want_big, o.score(big_model, big_graphs))
    # second call, straight after: a smaller input finds the first call's leftovers in the scratch
    want_small = small.score(2, 7, 4)
    got_small = score_static(small, 2, 7, 4)
    assert np.array_equal(got_small, want_small)
    assert np.array_equal(want_small, o.score(small_model, small_graphs, range(2, 9)))
    # and the first again, after the smaller one
    assert np.array_equal(score_static(big, 0, 60, 16), want_big)
    # what the entry point is for: its calls leave the device's free memory as it was (the output
    # tensors exist before the first reading; torch's allocator is not asked for anything in between),
    # also while launch timing is switched on - this entry point records no events
    out_big = torch.empty(60 * big.cfg.classes, dtype=torch.int32, device="cuda")
    out_small = torch.empty(7 * small.cfg.classes, dtype=torch.int32, device="cuda")
    st_big, st_small = big.state(), small.state()
    torch.cuda.synchronize()
    _abi.call("gtm_profile_enable", 1)
    try:
        free_before = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            _abi.call("gtm_score_static", ctypes.byref(big.acfg), ctypes.byref(big.dg.desc), ctypes.byref(st_big), 0, 60,
                      16, _ptr(out_big), _stream())
            _abi.call("gtm_score_static", ctypes.byref(small.acfg), ctypes.byref(small.dg.desc), ctypes.byref(st_small),
                      2, 7, 4, _ptr(out_small), _stream())
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
        _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
        assert launches.value == 0  # nothing was timed, and the switch is still on for other callers:
        big.score(0, 60, 16)
        _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
        assert launches.value > 0
    finally:
        _abi.call("gtm_profile_enable", 0)
    assert np.array_equal(out_big.cpu().numpy().reshape(60, -1), want_big)
    assert np.array_equal(out_small.cpu().numpy().reshape(7, -1), want_small)


def test_sizes_beyond_the_static_scratch_are_refused():
    dev, _, _ = device(500, 2, n_graphs=40, max_nodes=90, clauses=300, classes=4, tiles=False)
    need = _abi.lib.gtm_score_workspace_bytes(ctypes.byref(dev.acfg), ctypes.byref(dev.dg.desc), 1 << 20)
    assert need > _abi.lib.gtm_score_static_scratch_bytes()
    out = torch.zeros(40 * 4, dtype=torch.int32, device="cuda")
    st = dev.state()
    with pytest.raises(_abi.GtmError, match="allocation-free entry point has"):
        _abi.call("gtm_score_static", ctypes.byref(dev.acfg), ctypes.byref(dev.dg.desc), ctypes.byref(st), 0, 40,
                  1 << 20, _ptr(out), _stream())
    assert not out.any().item()  # nothing ran
