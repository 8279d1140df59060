"""Pins the oracle's ShowDecay / DeleteByShow restatement
(ada_grad_kernel.cc:191-204, ftrl_kernel.cc:124-126, adam_kernel.h:67-69) with
known answers and closed forms."""
import numpy as np
import pytest

from oracle import cpu as oracle


def table(kind, **hyper):
    t = oracle.Table(kind, 4, buckets=1 << 10, **hyper)
    signs = np.arange(1, 5, dtype=np.uint64)
    w = np.zeros((4, t.wf), np.float32)
    st = np.zeros((4, t.sf), np.float32)
    return t, signs, w, st


def test_adagrad_decay_known_answer_and_closed_form():
    t, signs, w, st = table(oracle.ADAGRAD, show_decay_rate=0.5, show_threshold=3.0, no_show_days=2)
    st[:, 1] = [16, 8, 4, 2]        # show
    st[:, 2] = [8, 4, 2, 1]         # click
    st[:, 3] = np.array([0, 1, 2, 3], np.int32).view(np.float32)  # no_show_days
    t.set_rows(signs, w, st)
    assert t.delete_by_show(signs).tolist() == [False, False, False, True]   # show < 3 or days > 2
    t.show_decay(1)
    _, s1, _ = t.get_rows(signs)
    assert s1[:, 1].tolist() == [8, 4, 2, 1] and s1[:, 2].tolist() == [4, 2, 1, 0.5]
    assert s1[:, 3].view(np.int32).tolist() == [1, 2, 3, 4]
    assert t.delete_by_show(signs).tolist() == [False, False, True, True]
    for _ in range(3):
        t.show_decay(2)
    _, s4, _ = t.get_rows(signs)
    np.testing.assert_array_equal(s4[:, 1], st[:, 1] * 0.5 ** 4)              # show * rate^k, exact for powers of two
    assert s4[:, 3].view(np.int32).tolist() == [7, 8, 9, 10]                  # days + sum of deltas
    assert t.delete_by_show(np.array([99], np.uint64)).tolist() == [False]    # absent sign


def test_adagrad_elimination_logic_and():
    t, signs, w, st = table(oracle.ADAGRAD, show_threshold=3.0, no_show_days=2, elimination_logic=1)
    st[:, 1] = [16, 1, 16, 1]
    st[:, 3] = np.array([0, 0, 5, 5], np.int32).view(np.float32)
    t.set_rows(signs, w, st)
    assert t.delete_by_show(signs).tolist() == [False, False, False, True]   # show < 3 and days > 2


def test_ftrl_and_adam():
    t, signs, w, st = table(oracle.FTRL, show_decay_rate=0.25, show_threshold=1.0)
    st[:, 8] = [16, 4, 2, 0.5]      # show sits after z[4], n[4]
    t.set_rows(signs, w, st)
    assert t.delete_by_show(signs).tolist() == [False, False, False, True]
    t.show_decay(7)
    _, s1, _ = t.get_rows(signs)
    assert s1[:, 8].tolist() == [4, 1, 0.5, 0.125]
    assert (s1[:, :8] == 0).all() and (s1[:, 9].view(np.int32) == 0).all()    # nothing else moves
    assert t.delete_by_show(signs).tolist() == [False, False, True, True]
    a, signs, w, st = table(oracle.ADAM, show_decay_rate=0.5, show_threshold=100.0)
    st[:, 8] = [16, 4, 2, 0.5]
    a.set_rows(signs, w, st)
    a.show_decay(3)
    _, s2, _ = a.get_rows(signs)
    assert (s2 == st).all() and not a.delete_by_show(signs).any()             # Adam: no decay, never eliminated
