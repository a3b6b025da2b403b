"""Saturating counters, Type I / II feedback, feedback gating and node
selection of the oracle, pinned by closed forms on decoded integer states,
exhaustive enumeration and distribution checks."""

import numpy as np
import pytest

from oracle import gtm_oracle as o


def decode(bank):
    """bit planes -> integer state per automaton, shape [C][chunks][32]."""
    C, W, B = bank.shape
    lanes = np.arange(32, dtype=np.uint32)
    bits = (bank[:, :, :, None] >> lanes) & 1  # [C][W][B][32]
    weights = (1 << np.arange(B, dtype=np.int64))[None, None, :, None]
    return (bits.astype(np.int64) * weights).sum(axis=2)


def encode(states, B):
    C, W, _ = states.shape
    bank = np.zeros((C, W, B), dtype=np.uint32)
    for b in range(B):
        plane = ((states >> b) & 1).astype(np.uint64)
        bank[:, :, b] = (plane << np.arange(32, dtype=np.uint64)).sum(axis=2).astype(np.uint32)
    return bank


@pytest.mark.parametrize("B", [1, 2, 4, 8, 10])
def test_inc_dec_exhaustive(B):
    """Every state x {active, inactive}: inc = min(s+1, 2^B-1), dec = max(s-1, 0)."""
    n_states = 1 << B
    per_word = 16  # 16 states x (active | inactive) fill one 32-lane word
    words = (n_states + per_word - 1) // per_word
    states = np.zeros((1, words, 32), dtype=np.int64)
    active = np.zeros((1, words), dtype=np.uint32)
    for s in range(n_states):
        w, lane = s // per_word, (s % per_word) * 2
        states[0, w, lane] = s
        states[0, w, lane + 1] = s
        active[0, w] |= np.uint32(1 << lane)
    on = ((active[:, :, None] >> np.arange(32, dtype=np.uint32)) & 1).astype(bool)
    up = encode(states, B)
    o.inc(up, active)
    assert np.array_equal(decode(up), np.where(on, np.minimum(states + 1, n_states - 1), states))
    down = encode(states, B)
    o.dec(down, active)
    assert np.array_equal(decode(down), np.where(on, np.maximum(states - 1, 0), states))


def unpack_words(words):
    return ((words[..., None] >> np.arange(32, dtype=np.uint32)) & 1).astype(bool)


def setup_feedback(seed, clauses=30, chunks=3, B=8, classes=3, literals=80, max_included=None, boost=1):
    rng = np.random.default_rng(seed)
    cfg = o.Config(classes=classes, clauses=clauses, literals=literals, state_bits=B, max_nodes=4,
                   boost_true_positive_feedback=boost, max_included_literals=max_included)
    states = rng.integers(0, 1 << B, size=(clauses, chunks, 32))
    rows = rng.integers(0, 2**32, size=(4, chunks), dtype=np.uint64).astype(np.uint32)
    clause_node = rng.integers(-1, 4, size=clauses).astype(np.int32)
    n_incl = rng.integers(0, 10, size=clauses).astype(np.int32)
    return cfg, rng, states, rows, clause_node, n_incl


@pytest.mark.parametrize("boost", [0, 1])
def test_type_one_feedback_closed_form(boost):
    """One class with update +1.  With s = 1 every feedback bit is 1, so Type I is
    deterministic: fired clauses do +1 on true literals (boost) / nothing
    (no boost, x & ~fb = 0) and -1 on false ones; others do -1 everywhere."""
    cfg, rng, states, rows, clause_node, n_incl = setup_feedback(1, classes=1, max_included=5, boost=boost)
    bank = encode(states, 8)
    upd = np.ones((1, cfg.clauses), dtype=np.int32)
    o.update(cfg, 7, 3, 1.0, bank, clause_node, n_incl, rows, upd)
    fired = clause_node != -1
    within = n_incl <= 5
    x = np.zeros((cfg.clauses, 3, 32), dtype=bool)
    x[fired] = unpack_words(rows)[clause_node[fired]]
    want = states.copy()
    good = (fired & within)[:, None, None]
    if boost:
        want = np.where(good & x, np.minimum(want + 1, 255), want)
    want = np.where(good & ~x, np.maximum(want - 1, 0), want)
    want = np.where(~good, np.maximum(want - 1, 0), want)
    assert np.array_equal(decode(bank), want)


def test_type_one_uses_the_feedback_bits_for_general_s():
    cfg, rng, states, rows, clause_node, n_incl = setup_feedback(2, classes=2, boost=0)
    bank = encode(states, 8)
    upd = np.zeros((2, cfg.clauses), dtype=np.int32)
    upd[1] = 1
    s = 4.0
    o.update(cfg, 11, 9, s, bank, clause_node, n_incl, rows, upd)
    fb = unpack_words(o.feedback_bits(11, 9, 0, 1, cfg.clauses, 3, o.feedback_threshold(s)))
    fired = (clause_node != -1)[:, None, None]
    x = np.zeros((cfg.clauses, 3, 32), dtype=bool)
    x[clause_node != -1] = unpack_words(rows)[clause_node[clause_node != -1]]
    want = states.copy()
    want = np.where(fired & x & ~fb, np.minimum(want + 1, 255), want)  # boost off: inc(x & ~fb)
    want = np.where(fired & ~x & fb, np.maximum(want - 1, 0), want)
    want = np.where(~fired & fb, np.maximum(want - 1, 0), want)
    assert np.array_equal(decode(bank), want)


def test_type_two_feedback_closed_form():
    """update -1 on a fired clause: +1 on literals that are 0 and not included."""
    cfg, rng, states, rows, clause_node, n_incl = setup_feedback(3, classes=1)
    bank = encode(states, 8)
    upd = -np.ones((1, cfg.clauses), dtype=np.int32)
    o.update_message(cfg, 1, 2, 1, 3.0, bank, clause_node, n_incl, rows, upd)
    fired = clause_node != -1
    x = np.zeros((cfg.clauses, 3, 32), dtype=bool)
    x[fired] = unpack_words(rows)[clause_node[fired]]
    included = states >= 128
    want = np.where(fired[:, None, None] & ~x & ~included, states + 1, states)
    assert np.array_equal(decode(bank), want)


def test_classes_apply_in_order_to_the_same_bank():
    """Type II after Type I sees the include plane Type I left behind."""
    cfg = o.Config(classes=2, clauses=1, literals=32, state_bits=8, max_nodes=1)
    states = np.full((1, 1, 32), 127, dtype=np.int64)
    rows = np.array([[0x0000FFFF]], dtype=np.uint32)
    node = np.zeros(1, dtype=np.int32)
    n_incl = np.zeros(1, dtype=np.int32)
    bank = encode(states, 8)
    o.update(cfg, 5, 0, 1.0, bank, node, n_incl, rows, np.array([[1], [-1]], dtype=np.int32))
    # class 0 (Type I, s=1): lanes 0-15 -> 128 (now included), lanes 16-31 -> 126
    # class 1 (Type II): lanes 16-31 are 0 and excluded -> back to 127
    assert np.array_equal(decode(bank)[0, 0], [128] * 16 + [127] * 16)
    bank = encode(states, 8)
    o.update(cfg, 5, 0, 1.0, bank, node, n_incl, rows, np.array([[-1], [1]], dtype=np.int32))
    assert np.array_equal(decode(bank)[0, 0], [128] * 16 + [127] * 16)
    bank = encode(states, 8)
    o.update(cfg, 5, 0, 1.0, bank, -np.ones(1, dtype=np.int32), n_incl, rows, np.array([[-1], [0]], dtype=np.int32))
    assert np.array_equal(decode(bank), states)  # Type II needs a fired clause


def test_initial_weights_are_a_fair_coin():
    """kernels.py:646-652: `1 - 2 * (curand % 2)` is +1 or -1 with equal probability, independently per
    (class, clause).  Over 10 x 20,000 weights the mean stays within 5 standard errors of 0, so do the
    means of every class row, neighbouring clauses are uncorrelated, and another seed gives another
    draw; with NEGATIVE_CLAUSES == 0 every weight is 1."""
    cfg = o.Config(classes=10, clauses=20000, literals=8, threshold=10)
    _, w = o.prepare(cfg, seed=42)
    assert w.shape == (10, 20000) and w.dtype == np.int32
    assert set(np.unique(w)) == {-1, 1}
    n = w.size
    assert abs(w.mean()) < 5.0 / np.sqrt(n)
    assert np.all(np.abs(w.mean(axis=1)) < 5.0 / np.sqrt(w.shape[1]))
    assert abs((w[:, 1:] * w[:, :-1]).mean()) < 5.0 / np.sqrt(n)   # clause c against clause c + 1
    assert abs((w[1:, :] * w[:-1, :]).mean()) < 5.0 / np.sqrt(n)   # class k against class k + 1
    _, other = o.prepare(cfg, seed=43)
    assert abs((w * other).mean()) < 5.0 / np.sqrt(n)
    _, later = o.prepare(cfg, seed=42, step=7)  # (the draw is addressed by the training step as well)
    assert abs((w * later).mean()) < 5.0 / np.sqrt(n)
    _, ones = o.prepare(o.Config(classes=3, clauses=50, literals=8, threshold=10, negative_clauses=0), seed=42)
    assert np.array_equal(ones, np.ones((3, 50), dtype=np.int32))


def test_select_clause_updates_case_table():
    """Deterministic corners of kernels.py:371-402 (probabilities 0 and 1)."""
    T = 10
    cfg = o.Config(classes=2, clauses=4, literals=8, threshold=T, q=1.0, max_nodes=1)
    node = np.array([0, 0, -1, -1], dtype=np.int32)
    w = np.array([[3, -3, 3, -3], [2, -2, 0, -1]], dtype=np.int32)
    # class 0: y=+T, sum=-50 -> clipped -T, err=2T -> always update, target +1
    # class 1: y=-T, sum=-50 -> clipped -T = y, not above y -> target +1 but err=0 -> never update
    upd = o.select_clause_updates(cfg, 1, 1, w, np.array([-50, -50]), np.array([T, -T]), node)
    assert np.array_equal(upd, [[1, -1, 1, -1], [0, 0, 0, 0]])
    # only fired clauses move: update > 0 grows |W| (W += sign), update < 0 shrinks it (W -= sign)
    assert np.array_equal(w, [[4, -2, 3, -3], [2, -2, 0, -1]])
    # class 1: y=-T, sum=+50 -> clipped T > y -> target -1, err=2T, q/(K-1)=1 -> always update
    w = np.array([[3, -3, 3, -3], [2, -2, 0, -1]], dtype=np.int32)
    upd = o.select_clause_updates(cfg, 1, 1, w, np.array([50, 50]), np.array([T, -T]), node)
    assert np.array_equal(upd[1], [-1, 1, -1, 1])       # target * sign, W=0 counts as positive
    assert np.array_equal(upd[0], [0, 0, 0, 0])         # y=+T reached: err=0
    assert np.array_equal(w[1], [1, -3, 0, -1])         # W=2 votes against the target: shrinks; W=-2 agrees: grows


def test_weight_can_cross_zero_and_saturates():
    cfg = o.Config(classes=1, clauses=2, literals=8, threshold=5, max_nodes=1)
    w = np.array([[0, o.INT_MAX]], dtype=np.int32)
    node = np.zeros(2, dtype=np.int32)
    o.select_clause_updates(cfg, 1, 1, w, np.array([99]), np.array([-5]), node)  # target -1, update = -sign
    assert list(w[0]) == [-1, o.INT_MAX - 1]
    w = np.array([[0, o.INT_MAX]], dtype=np.int32)
    o.select_clause_updates(cfg, 1, 1, w, np.array([-99]), np.array([5]), node)  # target +1
    assert list(w[0]) == [1, o.INT_MAX]  # |W| < INT_MAX guard


def test_update_probability_follows_error_and_q():
    T, clauses = 100, 20000
    cfg = o.Config(classes=3, clauses=clauses, literals=8, threshold=T, q=0.5, max_nodes=1)
    node = np.zeros(clauses, dtype=np.int32)
    w = np.ones((3, clauses), dtype=np.int32)
    sums = np.array([40, 40, -100])
    y = np.array([T, -T, -T])
    upd = o.select_clause_updates(cfg, 77, 123, w, sums, y, node)
    rate = (upd != 0).mean(axis=1)
    # class 0: target +1, err 60 -> 60/200; class 1: target -1, err 140 -> (q/2) * 140/200; class 2: err 0
    for got, p in zip(rate, [0.30, 0.25 * 0.70, 0.0]):
        assert abs(got - p) <= 5 * np.sqrt(max(p * (1 - p), 1e-9) / clauses)
    assert (upd[0] >= 0).all() and (upd[1] <= 0).all()


def test_select_clause_node_is_uniform_over_true_nodes():
    clauses, n = 30000, 70
    cfg = o.Config(classes=2, clauses=clauses, literals=8, max_nodes=n)
    true_nodes = [3, 31, 32, 64, 69]
    bitmap = np.zeros((clauses, cfg.node_chunks), dtype=np.uint32)
    for t in true_nodes:
        bitmap[:, t // 32] |= np.uint32(1 << (t % 32))
    bitmap[::7] = 0  # some clauses are false everywhere
    bitmap[:, 2] |= np.uint32(0xFFFFFF00)  # garbage past the last node must not be picked
    picked = o.select_clause_node(cfg, 5, 8, bitmap, n)
    assert (picked[::7] == -1).all()
    rest = np.delete(picked, np.arange(0, clauses, 7))
    assert set(np.unique(rest)) == set(true_nodes)
    counts = np.array([(rest == t).sum() for t in true_nodes])
    expected = rest.size / len(true_nodes)
    assert ((counts - expected) ** 2 / expected).sum() < 25.0  # chi-square, 4 dof
    assert not np.array_equal(picked, o.select_clause_node(cfg, 5, 9, bitmap, n))


def test_noisy_xor_learns_like_the_reference_transcript():
    """README.md:156-161: ~(100 - noise) % train, 100 % test from the first epochs."""
    from graphtsetlinmachine_amd import workloads

    wl = workloads.noisy_xor(1500, 500)
    cfg = o.Config(classes=2, clauses=10, literals=64, threshold=100, max_nodes=2, message_size=256, message_bits=2)
    rng = np.random.default_rng(0)
    hv = np.stack([rng.choice(256, size=2, replace=False) for _ in range(10)]).astype(np.uint32)
    model = o.new_model(cfg, 2, 1.0, hv, seed=42)
    Y = o.encode_labels(wl.Y_train, 2, 100)
    o.fit(model, wl.graphs_train, Y, epochs=2)
    test_acc = (o.score(model, wl.graphs_test).argmax(axis=1) == wl.Y_test).mean()
    train_acc = (o.score(model, wl.graphs_train).argmax(axis=1) == wl.Y_train).mean()
    assert test_acc == 1.0
    assert train_acc >= 0.975
    assert model.step == 3000
