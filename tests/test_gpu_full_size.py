"""The 361-node convolutional configuration at its full test size (10,000 graphs, 2,500 clauses):
the C oracle on every graph, and properties that need no oracle at all.

* every class sum equals the C restatement's (a few thousand graphs/s on the host cores), a sample
  also the NumPy oracle's;
* scoring is a per-graph function: a shuffled subset of the graphs scores to the same rows, whatever
  tile a graph lands in;
* transform (per-operator kernels, clause/node bitmaps materialised) and score (tile kernels) agree:
  class sums identical, and the sums recomputed from the transformed clause outputs and the
  weights equal both;
* scoring twice gives the same result."""

import numpy as np
import pytest

from graphtsetlinmachine_amd import workloads
from oracle import gtm_oracle as o
from oracle import gtm_oracle_c as oc
from tests.test_gpu_model import oracle_twin

pytestmark = pytest.mark.gpu


def test_convolutional_configuration_at_full_test_size():
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.convolutional_images(n_train=8000, n_test=10000)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    test = wl.graphs_test
    sums = tm.score(test)
    assert sums.shape == (10000, 10)
    assert np.array_equal(tm.score(test), sums)
    assert (sums.argmax(axis=1) == wl.Y_test).mean() > 0.9

    # the oracle on a sample spread over the set (first and last tile included)
    model = oracle_twin(tm, wl.graphs_train)
    model.ta_state = tm.get_state()[0].reshape(model.ta_state.shape).copy()
    model.clause_weights = tm.get_weights().copy()
    model.cfg = oracle_twin(tm, test).cfg
    sample = [0, 1, 9, 10, 4999, 5003, 9989, 9999]
    assert np.array_equal(sums[sample], o.score(model, test, sample))
    assert np.array_equal(sums, oc.score(model, test, threads=min(16, oc.threads_available())))

    # a shuffled subset lands in other tiles and other slots
    rng = np.random.default_rng(7)
    picked = rng.permutation(10000)[:3001]
    assert np.array_equal(tm.score(test[picked]), sums[picked])

    # the bitmap path: same sums, and clause outputs that reproduce them through the weights
    part = test[np.arange(2000, 3000)]
    fired, part_sums = tm.transform(part)
    assert np.array_equal(part_sums, sums[2000:3000])
    assert np.array_equal(fired.astype(np.int64) @ tm.get_weights().T.astype(np.int64), part_sums)


def test_sequence_chains_at_full_test_size():
    """The same properties for a model with a message layer: 5,000 chains of 1,000 nodes."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.sequence_chains(n_train=300, n_test=5000)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    test = wl.graphs_test
    sums = tm.score(test)
    assert sums.shape == (5000, 2) and np.array_equal(tm.score(test), sums)

    state = tm.get_state()
    model = oracle_twin(tm, test)
    model.ta_state = state[0].reshape(model.ta_state.shape).copy()
    model.message_ta_state = [b.reshape(model.message_ta_state[0].shape).copy() for b in tm.save()["message_ta_state"]]
    model.clause_weights = tm.get_weights().copy()
    sample = [0, 1, 2, 2499, 4998, 4999]
    assert np.array_equal(sums[sample], o.score(model, test, sample))
    every_fifth = list(range(0, 5000, 5))
    assert np.array_equal(sums[every_fifth], oc.score(model, test, every_fifth, threads=min(16, oc.threads_available())))

    rng = np.random.default_rng(8)
    picked = rng.permutation(5000)[:1001]
    assert np.array_equal(tm.score(test[picked]), sums[picked])

    part = test[np.arange(1000, 1300)]
    fired, part_sums = tm.transform(part)
    assert np.array_equal(part_sums, sums[1000:1300])
    assert np.array_equal(fired.astype(np.int64) @ tm.get_weights().T.astype(np.int64), part_sums)


def test_training_at_full_model_size_follows_the_c_oracle():
    """2,500 clauses on 361-node graphs: the state after 400 examples from the initial state, bit for
    bit (the C restatement trains ~500 graphs/s on the host cores; the NumPy oracle needs minutes)."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.convolutional_images(n_train=400, n_test=64)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)  # initial state only
    model = oracle_twin(tm, wl.graphs_train)
    state = tm.get_state()
    assert np.array_equal(state[0], model.ta_state.reshape(-1)) and np.array_equal(
        state[1].reshape(model.clause_weights.shape), model.clause_weights)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    oc.fit(model, wl.graphs_train, o.encode_labels(wl.Y_train, tm.number_of_outputs, tm.T),
           threads=min(16, oc.threads_available()))
    state = tm.get_state()
    assert np.array_equal(state[1].reshape(model.clause_weights.shape), model.clause_weights)
    assert np.array_equal(state[0], model.ta_state.reshape(-1))
    assert np.array_equal(tm.score(wl.graphs_test), oc.score(model, wl.graphs_test))


@pytest.mark.parametrize("name,n_train", [("sequence_chains", 600), ("colour_convolution", 16), ("single_node_images", 600),
                                          ("noisy_xor", 3000), ("runs_of_a", 3000)])
def test_training_of_every_configuration_follows_the_c_oracle(name, n_train):
    """Each configuration at its full model size (the colour one: 8,000 clauses, three banks of
    2,048 literals, 841 nodes): the state after n_train examples from the initial state, bit for bit."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl = workloads.BUILDERS[name](n_train=n_train, n_test=8)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)  # initial state only
    model = oracle_twin(tm, wl.graphs_train)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True)
    oc.fit(model, wl.graphs_train, o.encode_labels(wl.Y_train, tm.number_of_outputs, tm.T),
           threads=min(16, oc.threads_available()))
    saved = tm.save()
    assert np.array_equal(saved["clause_weights"].reshape(model.clause_weights.shape), model.clause_weights)
    assert np.array_equal(saved["ta_state"], model.ta_state.reshape(-1))
    for got, want in zip(saved["message_ta_state"], model.message_ta_state):
        assert np.array_equal(got, want.reshape(-1))
    model.cfg = oracle_twin(tm, wl.graphs_test).cfg
    assert np.array_equal(tm.score(wl.graphs_test), oc.score(model, wl.graphs_test))


def test_a_whole_epoch_of_the_convolutional_configuration_follows_the_c_oracle(capsys):
    """All 60,000 training graphs of the 361-node configuration, one after the other: the state the
    benchmark times its scoring kernel on.  The GPU trains the epoch in 48 runs of 1,250 examples and
    its state is read back after each; the C restatement then goes from every one of those states
    over the next 1,250 examples (single-threaded, 16 runs side by side) and must arrive at the next
    state bit for bit.  The first state is the common initial one, so by induction the whole GPU
    trajectory is the oracle's - without the oracle having to do 60,000 examples in sequence."""
    import copy
    from concurrent.futures import ThreadPoolExecutor

    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    n, run = 60000, 1250
    wl = workloads.convolutional_images(n_train=n, n_test=512)
    np.random.seed(42)
    tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
    tm.fit(wl.graphs_train, wl.Y_train, epochs=0, incremental=True)  # initial state only
    first = oracle_twin(tm, wl.graphs_train)
    states = [tm.get_state()]
    assert np.array_equal(states[0][0], first.ta_state.reshape(-1))
    assert np.array_equal(states[0][1].reshape(first.clause_weights.shape), first.clause_weights)
    for start in range(0, n, run):
        tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True, examples=(start, run))
        states.append(tm.get_state())
    assert tm.step == n
    encoded = o.encode_labels(wl.Y_train, tm.number_of_outputs, tm.T)

    def follow(i):
        model = copy.copy(first)
        model.ta_state = states[i][0].reshape(first.ta_state.shape).copy()
        model.clause_weights = states[i][1].reshape(first.clause_weights.shape).copy()
        model.step = i * run
        oc.fit(model, wl.graphs_train, encoded, indices=range(i * run, (i + 1) * run), threads=1)
        return (np.array_equal(model.ta_state.reshape(-1), states[i + 1][0]) and
                np.array_equal(model.clause_weights.reshape(-1), states[i + 1][1].reshape(-1)))

    with ThreadPoolExecutor(max_workers=max(1, min(16, oc.threads_available()))) as pool:
        for i, same in enumerate(pool.map(follow, range(n // run))):
            assert same, "the GPU and the oracle part ways between examples %d and %d" % (i * run, (i + 1) * run)
            if i % 8 == 7:
                with capsys.disabled():
                    print(" [%d examples followed]" % ((i + 1) * run), end="", flush=True)
    last = copy.copy(first)
    last.ta_state = states[-1][0].reshape(first.ta_state.shape).copy()
    last.clause_weights = states[-1][1].reshape(first.clause_weights.shape).copy()
    sums = tm.score(wl.graphs_test)
    assert np.array_equal(sums, oc.score(last, wl.graphs_test, threads=min(16, oc.threads_available())))
    assert (sums.argmax(axis=1) == wl.Y_test).mean() > 0.95


TRAINED_COLOUR = {}


def trained_colour_state():
    """The colour configuration (8,000 clauses, three banks of 2,048 literals, 841 nodes, depth 3) after
    4,096 training examples on the GPU: clauses of a few dozen literals that still hold at many nodes,
    the regime the scoring and training kernels of this configuration spend their time in - a freshly
    initialised model (every clause empty) or one after a handful of examples (a thousand literals per
    clause) does not reach it.  Trained once per test session."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    if not TRAINED_COLOUR:
        wl = workloads.colour_convolution(n_train=4096 + 48, n_test=64)
        np.random.seed(42)
        tm = MultiClassGraphTsetlinMachine(**wl.params, seed=42)
        tm.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True, examples=(0, 4096))
        TRAINED_COLOUR.update(wl=wl, tm=tm, state=tm.save())
    return TRAINED_COLOUR["wl"], TRAINED_COLOUR["tm"], TRAINED_COLOUR["state"]


def oracle_at(tm, state, graphs):
    model = oracle_twin(tm, graphs)
    model.ta_state = state["ta_state"].reshape(model.ta_state.shape).copy()
    model.message_ta_state = [b.reshape(model.message_ta_state[0].shape).copy() for b in state["message_ta_state"]]
    model.clause_weights = state["clause_weights"].reshape(model.clause_weights.shape).copy()
    model.step = int(state["rng_step"])
    return model


@pytest.mark.parametrize("scoring", ["default", "rows-in-place", "full-walk", "messages-in-three-launches"])
def test_scoring_the_colour_configuration_at_a_trained_state(scoring, tune):
    """Every scoring path that this shape can take, on the trained state, against the C oracle."""
    wl, tm, state = trained_colour_state()
    included = np.unpackbits(state["ta_state"].reshape(8000, 64, 8)[:, :, 7].copy().view(np.uint8)).sum() / 8000
    assert 8 < included < 400, "not the regime this test is for: %.1f literals per clause" % included
    if scoring == "rows-in-place":
        tune("GTM_NO_HALF_ROWS", "1")    # layer 0 on all 2,050 rows read in place, candidates tested on their own words
    elif scoring == "full-walk":
        tune("GTM_NO_HALF_ROWS", "1")
        tune("GTM_NO_TWO_PHASE", "1")    # layer 0 as a walk of every literal's row
    elif scoring == "messages-in-three-launches":
        tune("GTM_MESSAGES_IN_LDS", "0")  # the vectors of what the nodes send and receive in global memory
    model = oracle_at(tm, state, wl.graphs_test)
    want = oc.score(model, wl.graphs_test, threads=min(16, oc.threads_available()))
    tm._test_graphs = None  # (the tiles are built per path)
    assert np.array_equal(tm.score(wl.graphs_test), want)
    assert len(np.unique(want.argmax(axis=1))) > 1  # the state tells classes apart


@pytest.mark.parametrize("training", ["one-launch", "one-launch-small-windows", "launches-per-example"])
def test_training_the_colour_configuration_from_a_trained_state(training, tune):
    """48 more examples from the trained state, on every training path this shape can take, against the
    C oracle: all three banks and the weights bit for bit, and the class sums afterwards."""
    from graphtsetlinmachine_amd.tm import MultiClassGraphTsetlinMachine

    wl, tm, state = trained_colour_state()
    if "model_after" not in TRAINED_COLOUR:
        model = oracle_at(tm, state, wl.graphs_train)
        oc.fit(model, wl.graphs_train, o.encode_labels(wl.Y_train, tm.number_of_outputs, tm.T),
               indices=range(4096, 4096 + 48), threads=min(16, oc.threads_available()))
        TRAINED_COLOUR["model_after"] = model
    model = TRAINED_COLOUR["model_after"]
    if training == "one-launch-small-windows":
        tune("GTM_FIT_DEEP_WINDOW_ROWS", "128")
    elif training == "launches-per-example":
        tune("GTM_NO_DEEP_PERSISTENT_FIT", "1")
    np.random.seed(42)
    again = MultiClassGraphTsetlinMachine(**wl.params, seed=1)
    again.load(state)
    assert again.step == 4096 and again.seed == 42
    again.fit(wl.graphs_train, wl.Y_train, epochs=1, incremental=True, examples=(4096, 48))
    saved = again.save()
    assert np.array_equal(saved["clause_weights"].reshape(model.clause_weights.shape), model.clause_weights)
    assert np.array_equal(saved["ta_state"], model.ta_state.reshape(-1))
    for got, want in zip(saved["message_ta_state"], model.message_ta_state):
        assert np.array_equal(got, want.reshape(-1))
    assert not np.array_equal(saved["ta_state"], state["ta_state"])  # the 48 examples did move the automata
    few = list(range(8))
    scorer = oracle_at(again, saved, wl.graphs_test)
    assert np.array_equal(again.score(wl.graphs_test)[few], oc.score(scorer, wl.graphs_test, few, threads=8))
