#!/usr/bin/env python3
"""Benchmark of the Graph Tsetlin Machine hot path on one MI355X.

A "step" is one pass of batched inference (clause evaluation per node ->
class sums) over the workload's test graphs, with the encoded graphs and the
model state already resident in HBM.  The model state comes from training on
the GPU for one epoch over a sample of the training graphs, so include masks
have a trained density rather than being empty.

Prints ONE JSON line (rank 0 / the only process).
"""

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
SETTLE = 30  # untimed scoring passes before every timed region's warm-up (see time_scoring)
STARTED = time.time()
VALU_PEAK_LANE_OPS = 256 * 64 * 2.4e9  # 32-bit integer lane operations per second

# Hardware counters of the scoring kernel on the convolutional workload (10,000 graphs per launch, state after
# one epoch), from rocprofv3 --pmc runs of this file; the summaries and the commands are under profiles/.
# FETCH_SIZE counts 2 KiB per unit and WRITE_SIZE 1 KiB per unit on this part (a 256 MiB copy kernel reads
# 131,087 and writes 262,144).  valu_busy = SQ_INSTS_VALU x 4 clocks / (4 SIMDs x SQ_BUSY_CU_CYCLES): the share of
# the clocks in which a CU has work in which its vector ALUs issue.  The figures belong to the kernel's source text as it was when they were taken: `source_sha256` is
# the hash of the text of the functions named in `functions` (kernel_source_hash below), and a run whose
# library was built from another text reports no counters rather than stale ones.
MEASURED_COUNTERS = {
    "convolutional_images": {
        "kernel": "k_tile_two_phase_half<score>", "commit": "f694c07",
        "functions": ("tile_segments_part", "lowest_bit_or_ones", "k_compile_clauses_half", "half_combine",
                      "k_tile_two_phase_half"),
        "source_sha256": "f53f163f2332f8e1e8a8475589e46d3e043090241be17a64c6dceac6a5b3cab0",
        "fetch_units": 113516.5, "write_units": 647.3, "valu_busy": 0.63, "graphs": 10000,
    },
}


def kernel_source_hash(functions, path=os.path.join(ROOT, "graphtsetlinmachine_amd", "csrc", "score_tiles.h")):
    """sha256 over the text of the named functions of score_tiles.h: each from the line that declares it
    (`... void name(` or `... name(` at the start of a definition) to the line of its closing brace in
    column 0.  White space at line ends is dropped; anything else that changes, changes the hash."""
    import hashlib
    import re

    lines = open(path).read().split("\n")
    h = hashlib.sha256()
    for name in functions:
        start = next(i for i, l in enumerate(lines)
                     if re.search(r"\b%s\(" % re.escape(name), l) and not l.startswith((" ", "//", "#")))
        end = next(i for i in range(start, len(lines)) if lines[i].startswith("}"))
        for l in lines[start:end + 1]:
            h.update(l.rstrip().encode() + b"\n")
    return h.hexdigest()


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--workload", default="convolutional_images")
    p.add_argument("--graphs", type=int, default=10000, help="test graphs scored per step")
    p.add_argument("--train-graphs", type=int, default=60000, help="training graphs used to produce the model state")
    p.add_argument("--train-epochs", type=int, default=1)
    p.add_argument("--cpu-sample", type=int, default=None, help="graphs timed on the CPU oracle")
    p.add_argument("--no-cpu", action="store_true")
    p.add_argument("--only-main", action="store_true", help="skip the short runs of the other four configurations")
    p.add_argument("--one-state", action="store_true", help="time the kernel on the headline state only")
    p.add_argument("--full-size", action="store_true", help="the chosen workload at its full data-set size: one epoch "
                   "of training on every training graph, every test graph scored, a sample spread over the set "
                   "(first and last tile, graphs on both sides of the 4 GiB mark of X) checked against the C oracle")
    p.add_argument("--copy-probe", action="store_true", help="only copy 256 MiB three times with a library copy kernel: "
                   "calibrates the units of the FETCH_SIZE / WRITE_SIZE counters under rocprofv3 --pmc")
    p.add_argument("--save-state", default="", help="write the trained model to this .npz file after the run")
    p.add_argument("--load-state", default="", help="score a model saved by --save-state instead of training one "
                   "(the process then runs the scoring path only: what a profiler should see)")
    return p.parse_args()


# (train graphs, test graphs) of the runs of the configurations that are not the main one: the sizes the
# configurations are stated with
OTHER_WORKLOADS = {
    "noisy_xor": (10000, 10000),
    "single_node_images": (60000, 10000),
    "convolutional_images": (60000, 10000),
    "sequence_chains": (20000, 5000),
    "colour_convolution": (50000, 10000),
}


def oracle_twin(tm, n_nodes):
    """The CPU oracle's model object holding the GPU model's current state."""
    from oracle import gtm_oracle as o

    state = tm.get_state()
    cfg = o.Config(classes=tm.number_of_outputs, clauses=tm.number_of_clauses, literals=tm.number_of_literals,
                   state_bits=tm.number_of_state_bits, threshold=tm.T, q=tm.q,
                   max_included_literals=tm.max_included_literals, max_nodes=n_nodes,
                   message_size=tm.message_size, message_bits=tm.message_bits)
    model = o.new_model(cfg, tm.depth, tm.s, tm.hypervectors, seed=tm.seed)
    model.ta_state = state[0].reshape(cfg.clauses, cfg.la_chunks, cfg.state_bits).copy()
    model.message_ta_state = [b.reshape(cfg.clauses, cfg.message_chunks, cfg.state_bits).copy()
                              for b in tm.message_ta_state]
    model.clause_weights = state[1].reshape(cfg.classes, cfg.clauses).copy()
    return model


def spread_sample(graphs):
    """Graphs spread over a data set: the first and last ones, the middle, and the graphs on both sides of
    every multiple of 4 GiB of literal words (where 32-bit offsets would wrap)."""
    import numpy as np

    n = graphs.number_of_graphs
    picks = {e for e in (0, 1, n // 2, n - 2, n - 1) if 0 <= e < n}
    words = graphs.X.shape[1]
    mark = (1 << 32) // (words * 4)  # nodes per 4 GiB of literal words
    for k in range(1, int(graphs.X.shape[0] // mark) + 1):
        g = int(np.searchsorted(graphs.node_index, k * mark, side="right")) - 1
        picks.update(e for e in (g - 1, g, g + 1) if 0 <= e < n)
    return sorted(picks)


def other_run(name, n_train, n_test, check_graphs, check_seconds=12.0):
    """One epoch of training and timed scoring passes on a configuration at its stated data-set size, with
    the roofline of its scoring kernels; a few class sums are checked against the NumPy oracle and, with the C
    restatement, every test graph - or, where that would take minutes (the C oracle needs about half a second
    per colour graph), a sample spread over the test and training sets."""
    import numpy as np
    import torch

    from graphtsetlinmachine_amd import workloads
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine
    from oracle import gtm_oracle as o
    from oracle import gtm_oracle_c as oc

    t0 = time.time()
    wl = workloads.BUILDERS[name](n_train=n_train, n_test=n_test)
    t_data = time.time() - t0
    print("bench.py: %s built in %.0f s (X: %.2f GB train, %.2f GB test)"
          % (name, t_data, wl.graphs_train.X.nbytes / 1e9, wl.graphs_test.X.nbytes / 1e9), file=sys.stderr, flush=True)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)
    torch.cuda.synchronize()
    t_train, train_kernels = timed_fit(tm, wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    tm.score_device(wl.graphs_test)  # uploads the test graphs
    torch.cuda.synchronize()
    # (a pass over the small test sets takes a millisecond or less: one call alone would time the call, not the GPU)
    run = time_scoring(tm, wl.graphs_test, steps=5, warmup=2, graphs=n_test)
    sums = run["sums"]
    roofline = roofline_of(tm, wl.graphs_test, run, steps=5, graphs=n_test)
    threads = max(1, min(16, oc.threads_available()))
    model = oracle_twin(tm, int(wl.graphs_test.max_number_of_graph_nodes))
    want = o.score(model, wl.graphs_test, range(check_graphs))
    t0 = time.perf_counter()
    # about 4 graphs per thread of the first call tell whether the whole test set fits the time
    probe = list(range(min(n_test, 4 * threads)))
    same = bool(np.array_equal(oc.score(model, wl.graphs_test, probe, threads=threads), sums[probe]))
    per_graph = (time.perf_counter() - t0) / len(probe)
    checked = {"test": len(probe)}
    if per_graph * n_test <= check_seconds:
        same = same and bool(np.array_equal(oc.score(model, wl.graphs_test, threads=threads), sums))
        checked = {"test": n_test}
    else:
        sums_train = tm.score_device(wl.graphs_train).cpu().numpy().reshape(n_train, -1)
        for label, graphs, got in (("test", wl.graphs_test, sums), ("train", wl.graphs_train, sums_train)):
            twin = oracle_twin(tm, int(graphs.max_number_of_graph_nodes))
            picks, done = spread_sample(graphs), []
            for at in range(0, len(picks), threads):
                if time.perf_counter() - t0 > check_seconds and done:
                    break
                part = picks[at:at + threads]
                same = same and bool(np.array_equal(oc.score(twin, graphs, part, threads=threads), got[part]))
                done += part
            checked[label + "_spread"] = done
    t_c = time.perf_counter() - t0
    n_checked = sum(v if isinstance(v, int) else len(v) for v in checked.values())
    return {
        "train_graphs": n_train, "test_graphs": n_test, "train_graphs_per_s": round(n_train / t_train, 1),
        "train_kernels": train_kernels,
        "inference_graphs_per_s": round(n_test * 5 / run["wall"], 1),
        "test_accuracy": round(float((sums.argmax(axis=1) == wl.Y_test).mean()), 4),
        "mean_included_literals": round(mean_included_literals(tm), 2),
        "roofline": roofline,
        "class_sums_equal_oracle_on": check_graphs if np.array_equal(want, sums[:check_graphs]) else "MISMATCH",
        "class_sums_equal_c_oracle_on": checked if same else "MISMATCH",
        "c_oracle_graphs_per_s": round(n_checked / t_c, 1), "c_oracle_threads": threads,
        "data_build_s": round(t_data, 1),
    }


FULL_SIZES = {  # (training graphs, test graphs) the configurations are stated with
    "noisy_xor": (10000, 10000), "single_node_images": (60000, 10000), "convolutional_images": (60000, 10000),
    "sequence_chains": (20000, 5000), "colour_convolution": (50000, 10000),
}


def full_size_run(name, check_seconds=60.0):
    """One epoch over every training graph and one scoring pass over every test graph of a configuration
    at its stated data-set size; the trained state goes to the C oracle, which scores a sample spread
    over both sets (first and last graphs, and graphs around every multiple of 4 GiB of X)."""
    import numpy as np
    import torch

    from graphtsetlinmachine_amd import workloads
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine
    from oracle import gtm_oracle_c as oc

    import threading

    n_train, n_test = FULL_SIZES[name]
    t0 = time.time()
    building = threading.Event()

    def heartbeat():  # building the largest data set takes minutes: say so while it lasts
        while not building.wait(30.0):
            print("bench.py: building %s ... %.0f s" % (name, time.time() - t0), file=sys.stderr, flush=True)

    threading.Thread(target=heartbeat, daemon=True).start()
    try:
        wl = workloads.BUILDERS[name](n_train=n_train, n_test=n_test)
    finally:
        building.set()
    t_data = time.time() - t0
    print("bench.py: %s built in %.0f s (X: %.2f GB train, %.2f GB test)"
          % (name, t_data, wl.graphs_train.X.nbytes / 1e9, wl.graphs_test.X.nbytes / 1e9), file=sys.stderr, flush=True)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    t0 = time.perf_counter()
    tm.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)  # upload, tiles, initial state
    torch.cuda.synchronize()
    t_upload = time.perf_counter() - t0
    t0 = time.perf_counter()
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    torch.cuda.synchronize()
    t_train = time.perf_counter() - t0
    print("bench.py: trained %d graphs in %.1f s" % (n_train, t_train), file=sys.stderr, flush=True)
    tm.score_device(wl.graphs_test)  # uploads the test graphs
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sums_test = tm.score_device(wl.graphs_test)
    torch.cuda.synchronize()
    t_test = time.perf_counter() - t0
    sums_test = sums_test.cpu().numpy().reshape(n_test, -1)
    t0 = time.perf_counter()
    sums_train = tm.score_device(wl.graphs_train)  # the training set is the one that crosses 4 GiB
    torch.cuda.synchronize()
    t_score_train = time.perf_counter() - t0
    sums_train = sums_train.cpu().numpy().reshape(n_train, -1)

    threads = max(1, min(16, oc.threads_available()))
    checked, same, t0 = {}, True, time.perf_counter()
    for label, graphs, sums in (("test", wl.graphs_test, sums_test), ("train", wl.graphs_train, sums_train)):
        model = oracle_twin(tm, int(graphs.max_number_of_graph_nodes))
        picks = spread_sample(graphs)
        done = []
        for at in range(0, len(picks), threads):  # bounded: a colour graph costs about half a second
            if time.perf_counter() - t0 > check_seconds and done:
                break
            part = picks[at:at + threads]
            same = same and bool(np.array_equal(oc.score(model, graphs, part, threads=threads), sums[part]))
            done += part
        checked[label] = done
    return {
        "workload": name, "train_graphs": n_train, "test_graphs": n_test,
        "X_train_bytes": int(wl.graphs_train.X.nbytes), "X_test_bytes": int(wl.graphs_test.X.nbytes),
        "total_train_nodes": int(wl.graphs_train.X.shape[0]),
        "train_graphs_per_s": round(n_train / t_train, 1), "inference_graphs_per_s": round(n_test / t_test, 1),
        "inference_graphs_per_s_on_the_training_set": round(n_train / t_score_train, 1),
        "test_accuracy": round(float((sums_test.argmax(axis=1) == wl.Y_test).mean()), 4),
        "class_sums_equal_c_oracle_on": checked if same else "MISMATCH",
        "data_build_s": round(t_data, 1), "upload_and_tiles_s": round(t_upload, 1),
    }


def eval_bytes_per_graph(n_nodes, la_chunks, clauses, node_chunks):
    """Algorithmic bytes of one layer-0 clause evaluation of one graph: its X
    rows, node types and the include plane in; the clause x node bitmap and the
    include counts out."""
    return n_nodes * la_chunks * 4 + n_nodes * 4 + clauses * la_chunks * 4 + clauses * node_chunks * 4 + clauses * 4


def read_kernel_profile():
    """(kernel name, launches, total ms) of the clause-evaluation kernel since
    profiling was enabled: HIP events recorded inside the library around each
    launch, on the stream the kernel runs on."""
    from graphtsetlinmachine_amd import _abi

    name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
    _abi.call("gtm_profile_read", ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
    return name.value.decode(), launches.value, total.value


def read_kernel_breakdown():
    """[(kernel name, launches, total ms)] for every kernel bracketed since profiling was enabled
    (read before read_kernel_profile(), which clears the record)."""
    from graphtsetlinmachine_amd import _abi

    out = []
    for index in range(64):
        name, launches, total = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_double()
        _abi.call("gtm_profile_read_kernel", index, ctypes.byref(name), ctypes.byref(launches), ctypes.byref(total))
        if not name.value:
            break
        out.append((name.value.decode(), launches.value, total.value))
    return out


def message_layer_bytes_per_graph(n_nodes, message_chunks, clauses, node_chunks, edges):
    """Algorithmic bytes of one message layer of one graph: the nodes' message literal words and the
    include plane of the layer's bank in, the edges walked once, the previous layer's clause x node
    bitmap in and the new one out."""
    return n_nodes * message_chunks * 4 + clauses * message_chunks * 4 + 2 * clauses * node_chunks * 4 + edges * 8


def roofline_of(tm, test, run, steps, graphs):
    """The roofline object of a timed scoring run (time_scoring): algorithmic bytes of the dominant kernel -
    or, for a model with message layers, of the group of kernels (layer 0 / the message layers) that takes
    longer - over that kernel's time, measured by the library's own events around each launch."""
    n_nodes = int(test.max_number_of_graph_nodes)
    la, node_chunks = tm.number_of_ta_chunks, (n_nodes - 1) // 32 + 1
    b_eval = eval_bytes_per_graph(n_nodes, la, tm.number_of_clauses, node_chunks)
    kernel_name, kernel_ms, launches = run["kernel"], run["kernel_ms"], run["launches"]
    graphs_per_launch = run["graphs_per_launch"]
    ms_per_step = run["wall"] * 1000.0 / steps
    layer_groups, step_bytes = None, b_eval
    if tm.depth > 1:
        edges_per_graph = int(test.edge.shape[0]) // max(int(test.number_of_graphs), 1)
        b_msg = message_layer_bytes_per_graph(n_nodes, tm.number_of_message_chunks, tm.number_of_clauses,
                                              node_chunks, edges_per_graph)
        layer_groups = []
        for label, wanted, group_bytes in (("layer 0", lambda k: "messages" not in k, b_eval),
                                          ("message layers (%d)" % (tm.depth - 1), lambda k: "messages" in k,
                                           b_msg * (tm.depth - 1))):
            members = [k for k in run["kernels"] if wanted(k["kernel"])]
            ms = sum(k["ms_per_step"] for k in members)
            gbs = group_bytes * graphs / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
            layer_groups.append({"layers": label, "kernels": [k["kernel"] for k in members], "ms_per_step": round(ms, 4),
                                 "algorithmic_bytes_per_graph": group_bytes, "achieved_GBs": round(gbs, 1),
                                 "frac": round(gbs / HBM_PEAK_GBS, 4)})
        step_bytes = sum(e["algorithmic_bytes_per_graph"] for e in layer_groups)
        slowest = max(layer_groups, key=lambda e: e["ms_per_step"])
        if slowest["ms_per_step"] > 0:
            b_eval, kernel_name = slowest["algorithmic_bytes_per_graph"], " + ".join(slowest["kernels"])
            kernel_ms, graphs_per_launch = slowest["ms_per_step"], float(graphs)
    timed = kernel_ms > 0
    achieved = b_eval * graphs_per_launch / (kernel_ms * 1e-3) / 1e9 if timed else None
    compulsory = (n_nodes * la * 4 + n_nodes * 4 + tm.number_of_outputs * 4) * graphs_per_launch
    return {
        "bound": "hbm", "achieved": round(achieved, 1) if timed else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4) if timed else None, "traffic": None,
        "kernel": kernel_name, "kernel_ms": round(kernel_ms, 4), "launches": launches,
        "graphs_per_launch": graphs_per_launch,
        "algorithmic_bytes_per_graph": b_eval,
        "kernels": run["kernels"], "layer_groups": layer_groups,
        # the same bytes (every layer's) over the whole timed step (kernels + clause compilation + launch gaps)
        "frac_whole_step": round(step_bytes * graphs / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        # what a batched kernel cannot avoid moving: the graphs' literal words and node types in, the class sums out
        "compulsory_GBs": round(compulsory / (kernel_ms * 1e-3) / 1e9, 1) if timed else None,
        # the dense formulation (one word test per clause, node and literal word) against the integer
        # VALU peak of 256 CUs x 64 lanes x 2.4 GHz: what a kernel that does not skip work could reach
        "dense_word_ops_per_graph": tm.number_of_clauses * n_nodes * la,
        "dense_valu_ceiling_graphs_per_s": round(VALU_PEAK_LANE_OPS / (tm.number_of_clauses * n_nodes * la), 1),
    }


def mean_included_literals(tm):
    import numpy as np

    bank = tm.get_state()[0].reshape(tm.number_of_clauses, tm.number_of_ta_chunks, tm.number_of_state_bits)
    plane = np.ascontiguousarray(bank[:, :, tm.number_of_state_bits - 1])
    return float(np.unpackbits(plane.view(np.uint8)).sum()) / tm.number_of_clauses


def timed_fit(tm, *fit_args, **fit_kwargs):
    """(seconds, [{kernel, launches, ms}]) of a call of tm.fit: wall clock around the call, and the library's own
    events around the training kernels it launched (one launch per call for the one-launch kernels)."""
    import torch

    from graphtsetlinmachine_amd import _abi

    _abi.call("gtm_profile_enable", 1)
    t0 = time.perf_counter()
    tm.fit(*fit_args, **fit_kwargs)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    kernels = [{"kernel": k, "launches": n, "ms": round(ms, 3)} for k, n, ms in read_kernel_breakdown()]
    read_kernel_profile()  # (clears the record)
    _abi.call("gtm_profile_enable", 0)
    return seconds, kernels


def time_scoring(tm, test, steps, warmup, graphs):
    """`steps` timed passes of gtm_score over the resident test graphs after `warmup` untimed ones."""
    import torch

    from graphtsetlinmachine_amd import _abi

    # The first launches after a stretch of other work (training, a CPU check) run at a lower clock: SETTLE
    # untimed passes come before the `warmup` passes that the caller asked for.
    for _ in range(SETTLE + warmup):
        tm.score_device(test)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    _abi.call("gtm_profile_enable", 1)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        sums = tm.score_device(test)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    breakdown = read_kernel_breakdown()
    kernel_name, launches, kernel_total_ms = read_kernel_profile()
    _abi.call("gtm_profile_enable", 0)
    if len(breakdown) > 1:  # several kernels share the work: the roofline kernel is the one that takes longest
        kernel_name, launches, kernel_total_ms = max(breakdown, key=lambda k: k[2])
    return {
        "kernels": [{"kernel": k, "launches_per_step": round(n / steps, 2), "ms_per_step": round(ms / steps, 4)}
                    for k, n, ms in breakdown],
        "wall": wall, "event_ms": start.elapsed_time(stop) / steps, "kernel": kernel_name, "launches": launches,
        "kernel_ms": kernel_total_ms / max(launches, 1), "graphs_per_launch": graphs * steps / max(launches, 1),
        "sums": sums.cpu().numpy().reshape(graphs, -1),
    }


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; inference shards by graph range and training by clause, "
              "but no multi-GPU path is part of it. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    if args.copy_probe:
        a = torch.empty(256 * 1024 * 1024 // 4, dtype=torch.int32, device="cuda").fill_(1)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        print("copied %d bytes three times" % (a.numel() * 4))
        return

    from graphtsetlinmachine_amd import workloads
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    torch.cuda.set_device(0)
    if args.full_size:
        result = full_size_run(args.workload)
        print(json.dumps({"metric": "train & inference graphs/sec on 1 MI355X (%s at full data-set size)" % args.workload,
                          "value": result["inference_graphs_per_s"], "unit": "graphs/s", "n_gpus": 1,
                          "higher_is_better": True, "dtype": "u32", "data": "synthetic",
                          "config": {"workload": args.workload}, "full_size": result}), flush=True)
        if result["class_sums_equal_c_oracle_on"] == "MISMATCH":
            print("bench.py: GPU class sums differ from the C oracle", file=sys.stderr)
            sys.exit(1)
        return
    t0 = time.time()
    wl = workloads.BUILDERS[args.workload](n_train=args.train_graphs, n_test=args.graphs)
    t_data = time.time() - t0
    test = wl.graphs_test
    n_nodes = int(test.max_number_of_graph_nodes)

    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    if args.load_state:
        import contextlib

        with contextlib.redirect_stdout(sys.stderr):  # load() announces the file, as the reference's does
            tm.load(fname=args.load_state)
        args.one_state, args.train_epochs = True, 0
    else:
        tm.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)  # allocate + upload only
    tm.score_device(test)  # uploads the test graphs
    torch.cuda.synchronize()
    la = tm.number_of_ta_chunks
    b_eval = eval_bytes_per_graph(n_nodes, la, tm.number_of_clauses, (n_nodes - 1) // 32 + 1)

    def frac_of(run):
        return b_eval * run["graphs_per_launch"] / (run["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS

    def c_oracle_agrees(run):
        from oracle import gtm_oracle_c as oc

        model = oracle_twin(tm, n_nodes)
        return bool(np.array_equal(oc.score(model, test, threads=max(1, min(16, oc.threads_available()))), run["sums"]))

    def state_entry(label, run, checked):
        return {"state": label, "frac": round(frac_of(run), 4), "kernel_ms": round(run["kernel_ms"], 4),
                "graphs_per_s": round(args.graphs * args.steps / run["wall"], 1),
                "mean_included_literals": round(mean_included_literals(tm), 2),
                "class_sums_equal_c_oracle": checked}

    # The include density of the state decides how much the sparse kernel can skip, so the kernel is
    # timed on three states of the same run: early in the first epoch, after the configured epochs
    # (the headline, `value`), and after two epochs more.
    states = []
    early = min(5000, args.train_graphs // 2)
    t_train, train_kernels = 0.0, []
    if early > 0 and args.train_epochs >= 1 and not args.one_state:
        t0 = time.time()
        tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True, examples=(0, early))
        torch.cuda.synchronize()
        t_train += time.time() - t0
        run = time_scoring(tm, test, args.steps, args.warmup, args.graphs)
        states.append(state_entry("after %d training graphs" % early, run, None if args.no_cpu else c_oracle_agrees(run)))
        seconds, train_kernels = timed_fit(tm, wl.graphs_train, wl.Y_train, epochs=1, incremental=True,
                                           examples=(early, args.train_graphs - early))
        t_train += seconds
        if args.train_epochs > 1:
            t_train += timed_fit(tm, wl.graphs_train, wl.Y_train, epochs=args.train_epochs - 1, incremental=True)[0]
    elif not args.load_state:
        t_train, train_kernels = timed_fit(tm, wl.graphs_train, wl.Y_train, epochs=args.train_epochs, incremental=True)
    train_gps = args.train_graphs * args.train_epochs / max(t_train, 1e-9)
    if args.save_state:
        import contextlib

        with contextlib.redirect_stdout(sys.stderr):
            tm.save(args.save_state)

    main_run = time_scoring(tm, test, args.steps, args.warmup, args.graphs)
    wall, kernel_name, launches = main_run["wall"], main_run["kernel"], main_run["launches"]
    kernel_ms, graphs_per_launch, event_ms = main_run["kernel_ms"], main_run["graphs_per_launch"], main_run["event_ms"]
    sums_host = main_run["sums"]
    ms_per_step = wall * 1000.0 / args.steps
    value = args.graphs * args.steps / wall
    accuracy = float((sums_host.argmax(axis=1) == wl.Y_test).mean())
    included_main = mean_included_literals(tm)

    roofline = roofline_of(tm, test, main_run, args.steps, args.graphs)
    kernel_name, kernel_ms, graphs_per_launch = roofline["kernel"], roofline["kernel_ms"], roofline["graphs_per_launch"]
    # what the memory system really moved (rocprofv3 FETCH_SIZE + WRITE_SIZE) over this run's kernel time, and the
    # share of cycles in which the vector ALUs issued: from the counter runs named at the top of this file, and
    # only while the kernel's source text is the one they were taken on
    counters = MEASURED_COUNTERS.get(args.workload)
    if counters and (counters["kernel"] != kernel_name or
                     counters["source_sha256"] != kernel_source_hash(counters["functions"])):
        counters = None
    traffic = (round((counters["fetch_units"] * 2 + counters["write_units"]) * 1024 / counters["graphs"] * graphs_per_launch)
               if counters else None)
    roofline.update({
        "traffic": traffic,
        "hbm_measured_GBs": round(traffic / (kernel_ms * 1e-3) / 1e9, 1) if traffic else None,
        "hbm_measured_frac": round(traffic / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if traffic else None,
        "valu_busy": counters["valu_busy"] if counters else None,
        "counters_measured_at_commit": counters["commit"] if counters else None,
    })

    cpu = None
    if not args.no_cpu:
        from oracle import gtm_oracle as o
        from oracle import gtm_oracle_c as oc

        model = oracle_twin(tm, n_nodes)
        # the C restatement of the reference's kernels on the box's host cores: whole passes over the
        # step's graphs for about 10 s, every class sum compared with the GPU's
        threads = max(1, min(16, oc.threads_available()))
        passes, t0 = 0, time.perf_counter()
        while True:
            want = oc.score(model, test, threads=threads)
            passes += 1
            t_cpu = time.perf_counter() - t0
            if t_cpu >= 10.0 or passes >= 200:
                break
        if not np.array_equal(want, sums_host):
            print("bench.py: GPU class sums differ from the C oracle", file=sys.stderr)
            sys.exit(1)
        rate = passes * args.graphs / t_cpu
        # one thread, about 3 s
        one = max(8, min(args.graphs, int(3.0 * rate / threads)))
        t0 = time.perf_counter()
        oc.score(model, test, range(one), threads=1)
        t_one = time.perf_counter() - t0
        # the NumPy oracle (~3.5 ns per clause x node x word) as a second opinion, about 3 s
        sample = args.cpu_sample or max(8, int(3.0 / (tm.number_of_clauses * n_nodes * la * tm.depth * 3.5e-9)))
        sample = min(sample, args.graphs)
        t0 = time.perf_counter()
        want_np = o.score(model, test, range(sample))
        t_np = time.perf_counter() - t0
        if not np.array_equal(want_np, sums_host[:sample]):
            print("bench.py: GPU class sums differ from the NumPy oracle on the sample", file=sys.stderr)
            sys.exit(1)
        # training: the C restatement continuing from the GPU model's state for about 5 s (16 threads at
        # most: clauses of one example in parallel, examples one after the other), and the NumPy oracle
        # on a few graphs
        train_model = oracle_twin(tm, int(wl.graphs_train.max_number_of_graph_nodes))
        encoded_all = o.encode_labels(wl.Y_train, tm.number_of_outputs, tm.T)
        trained, t0 = 0, time.perf_counter()
        while trained < args.train_graphs and time.perf_counter() - t0 < 5.0:
            upto = min(args.train_graphs, trained + 64)
            oc.fit(train_model, wl.graphs_train, encoded_all, indices=range(trained, upto), threads=threads)
            trained = upto
        t_c_train = time.perf_counter() - t0
        train_sample = max(2, min(sample // 2, args.train_graphs))
        train_model = oracle_twin(tm, int(wl.graphs_train.max_number_of_graph_nodes))
        t0 = time.perf_counter()
        o.fit(train_model, wl.graphs_train, encoded_all, indices=range(train_sample))
        t_cpu_train = time.perf_counter() - t0
        cpu = {"value": round(rate, 1), "unit": "graphs/s", "cores": threads, "kind": "port",
               "sample": "C restatement of the reference's kernels (oracle/gtm_oracle.c, OpenMP over graphs): %d "
                         "pass(es) over the step's %d graphs in %.1f s, every class sum equal to the GPU's"
                         % (passes, args.graphs, t_cpu),
               "one_core_value": round(one / t_one, 1),
               "numpy_value": round(sample / t_np, 2),
               "numpy_sample": "NumPy oracle on the first %d graphs (%.1f s), equal to the GPU sums" % (sample, t_np),
               "train_value": round(trained / t_c_train, 1),
               "train_sample": "C restatement, %d threads, %d training graphs one after the other (%.1f s)"
                               % (threads, trained, t_c_train),
               "numpy_train_value": round(train_sample / t_cpu_train, 2),
               "numpy_train_sample": "NumPy oracle, one training pass over %d graphs (%.1f s)"
                                     % (train_sample, t_cpu_train)}

    if states:
        states.append({"state": "after %d epoch(s) (the headline)" % args.train_epochs, "frac": roofline["frac"],
                       "kernel_ms": roofline["kernel_ms"], "graphs_per_s": round(value, 1),
                       "mean_included_literals": round(included_main, 2),
                       "class_sums_equal_c_oracle": None if args.no_cpu else True})
        tm.fit(wl.graphs_train, wl.Y_train, epochs=2, incremental=True)
        torch.cuda.synchronize()
        run = time_scoring(tm, test, args.steps, args.warmup, args.graphs)
        states.append(state_entry("after %d epochs" % (args.train_epochs + 2), run,
                                  None if args.no_cpu else c_oracle_agrees(run)))
        roofline["states"] = states
        roofline["frac_worst_state"] = min(e["frac"] for e in states)
        if any(e["class_sums_equal_c_oracle"] is False for e in states):
            print("bench.py: GPU class sums differ from the C oracle on a state: %s" % json.dumps(states), file=sys.stderr)
            sys.exit(1)

    others = {}
    if not args.only_main:
        for name, (n_train, n_test) in OTHER_WORKLOADS.items():
            if name == args.workload:
                continue
            if name == "colour_convolution" and time.time() - STARTED > 300.0:
                # its 10.8 GB data set takes about a minute to build and the run two more: not on top of a run
                # that is already slow (a loaded host), or the whole line is lost to the caller's time limit
                n_train, n_test = n_train // 10, n_test // 10
            others[name] = other_run(name, n_train, n_test, check_graphs=2 if name == "colour_convolution" else 16)
            print("bench.py: %s done" % name, file=sys.stderr, flush=True)
        if "noisy_xor" in others:
            # the only rates the reference publishes (its README transcript of this demo, 10,000 + 10,000
            # graphs, hardware not stated): 1.52-1.55 s per training epoch, 0.88 s per test pass
            others["noisy_xor"]["reference_readme_train_graphs_per_s"] = 6500
            others["noisy_xor"]["reference_readme_test_graphs_per_s"] = 11400
        wrong = [name for name, r in others.items()
                 if "MISMATCH" in (r["class_sums_equal_oracle_on"], r["class_sums_equal_c_oracle_on"])]
        if wrong:
            print("bench.py: GPU class sums differ from a CPU oracle on %s: %s"
                  % (", ".join(wrong), json.dumps({n: others[n] for n in wrong})), file=sys.stderr)
            sys.exit(1)

    line = {
        "metric": "inference graphs/sec on 1 MI355X (%s)" % args.workload,
        "value": round(value, 1), "unit": "graphs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32", "data": "synthetic",
        "config": {"workload": args.workload, "graphs_per_step": args.graphs, "nodes_per_graph": n_nodes,
                   "clauses": tm.number_of_clauses, "literals": tm.number_of_literals, "depth": tm.depth,
                   "classes": tm.number_of_outputs,
                   "state": ("loaded from %s" % args.load_state) if args.load_state else
                            "trained %d epoch(s) on %d graphs on the GPU" % (args.train_epochs, args.train_graphs),
                   "mean_included_literals": round(included_main, 2),
                   "untimed_passes_before_warmup": SETTLE},
        "roofline": roofline, "cpu_baseline": cpu,
        "train_graphs_per_s": round(train_gps, 1), "train_kernels": train_kernels, "test_accuracy": round(accuracy, 4),
        "event_ms_per_step": round(event_ms, 4), "data_build_s": round(t_data, 1),
        "other_workloads": others,
    }
    print(json.dumps(line), flush=True)
    # nothing of this process's is left on the device when the interpreter starts to shut down
    del tm, wl, test
    import gc

    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
