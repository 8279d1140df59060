"""Pins the oracle's restatement of the checkpoint streams (optimizer_kernel.h:324-420,
ada_grad_kernel.cc:131-189, adam_kernel.cc:127-167, ftrl_kernel.cc:82-122) with hand-written
files and byte layouts."""
import struct

import numpy as np
import pytest

from oracle import cpu as oracle


def small(kind, **hyper):
    t = oracle.Table(kind, 2, buckets=1 << 10, **hyper)
    signs = np.array([8, 16], np.uint64)   # (s >> 32 | s << 32) % 8 == 0: both in block 0
    return t, signs


def test_adagrad_txt_known_answer():
    t, signs = small(oracle.ADAGRAD, use_cvm=True)
    w = np.array([[0.5, -1.25, 0, 0], [1e-8, 3, 0, 0]], np.float32)
    st = np.array([[0.1, 3, 1, 0], [2, 7, 2, 0]], np.float32)
    st[:, 3] = np.array([4, 0], np.int32).view(np.float32)
    t.set_rows(signs, w, st)
    text = t.serialize_block(0, "txt").decode()
    assert text.startswith("opt_name:AdaGrad\ndim:2\n") and text.endswith("\n\n")
    rows = sorted(text.split("\n")[2:-2])
    assert rows == ["16\t2\t1e-08\t3\t2\t7\t0\t2", "8\t2\t0.5\t-1.25\t0.1\t3\t4\t1"]
    for b in range(1, 8):
        assert t.serialize_block(b, "txt") == b"opt_name:AdaGrad\ndim:2\n\n"


def test_adagrad_bin_layout_and_round_trip():
    t, signs = small(oracle.ADAGRAD, use_cvm=True)
    w = np.array([[0.5, -1.25, 0, 0], [1e-8, 3, 0, 0]], np.float32)
    st = np.array([[0.1, 3, 1, 0], [2, 7, 2, 0]], np.float32)
    st[:, 3] = np.array([4, 9], np.int32).view(np.float32)
    t.set_rows(signs, w, st)
    data = t.serialize_block(0, "bin")
    assert len(data) == 4 + 2 * (8 + 2 * 4 + 4 + 4 + 4 + 4) + 1 and data[-1:] == b"\n"
    assert struct.unpack_from("<i", data, 0) == (2,)
    recs = {}
    for k in range(2):
        sign, w0, w1, g2, show, days, click = struct.unpack_from("<Qffffif", data, 4 + k * 32)
        recs[sign] = (w0, w1, g2, show, days, click)
    assert recs[8] == (0.5, -1.25, np.float32(0.1), 3.0, 4, 1.0)
    assert recs[16] == (np.float32(1e-8), 3.0, 2.0, 7.0, 9, 2.0)
    t2, _ = small(oracle.ADAGRAD, use_cvm=True)
    assert t2.deserialize_block(data, "bin") == 2
    w2, s2, f2 = t2.get_rows(signs)
    assert f2.all() and (s2.view(np.int32) == st.view(np.int32)).all() and (w2[:, :2] == w[:, :2]).all()
    # the cvm columns are rebuilt from show / click on load (ada_grad_kernel.cc:181-186)
    np.testing.assert_allclose(w2[:, 2], st[:, 1])
    np.testing.assert_allclose(w2[:, 3], np.log(st[:, 2] + 1) - np.log(st[:, 1] + 1), rtol=1e-6)


def test_txt_round_trip_keeps_six_digits_and_old_files_load():
    t, signs = small(oracle.ADAGRAD)
    w = np.array([[0.123456789, -2.5], [3.0, 1e-3]], np.float32)
    st = np.array([[0.1, 3, 0, 0], [2, 7, 0, 0]], np.float32)
    st[:, 3] = np.array([4, 9], np.int32).view(np.float32)
    t.set_rows(signs, w, st)
    t2, _ = small(oracle.ADAGRAD)
    assert t2.deserialize_block(t.serialize_block(0, "txt"), "txt") == 2
    w2, s2, _ = t2.get_rows(signs)
    assert w2[0, 0] == np.float32(0.123457) and w2[0, 1] == np.float32(-2.5)       # %g: six significant digits
    assert (s2.view(np.int32)[:, 3] == [4, 9]).all() and s2[1, 1] == 7
    # a file written before no_show_days existed: dim + 4 columns (optimizer.h:107-112)
    old = b"opt_name:AdaGrad\ndim:2\n8\t2\t0.5\t-1.25\t0.25\t3\t\n16\t2\t1\t2\t0.5\t7\t\n\n"
    t3, _ = small(oracle.ADAGRAD)
    assert t3.deserialize_block(old, "txt") == 2
    w3, s3, _ = t3.get_rows(signs)
    assert w3.tolist() == [[0.5, -1.25], [1, 2]] and s3[:, :2].tolist() == [[0.25, 3], [0.5, 7]]
    assert (s3.view(np.int32)[:, 3] == 0).all()
    with pytest.raises(ValueError):          # written by another optimizer (optimizer_kernel.h:370-373)
        t3.deserialize_block(b"opt_name:Adam\ndim:2\n\n", "txt")


@pytest.mark.parametrize("kind,name", [(oracle.ADAM, "Adam"), (oracle.FTRL, "Ftrl")])
def test_adam_and_ftrl_formats(kind, name):
    t, signs = small(kind)
    w = np.array([[0.5, -1.25], [1, 2]], np.float32)
    st = np.array([[1, 2, 3, 4, 5, 0], [6, 7, 8, 9, 10, 0]], np.float32)   # a[2] b[2] show delta_show
    st[:, 5] = np.array([11, 12], np.int32).view(np.float32)
    t.set_rows(signs, w, st)
    rows = sorted(t.serialize_block(0, "txt").decode().split("\n")[2:-2])
    assert rows == ["16\t1\t6\t8\t2\t7\t9\t10", "8\t0.5\t1\t3\t-1.25\t2\t4\t5"]   # (w a b) per element, then show
    data = t.serialize_block(0, "bin")
    assert len(data) == 4 + 2 * (8 + 3 * 2 * 4 + 4) + 1
    t2, _ = small(kind)
    assert t2.deserialize_block(data, "bin") == 2
    w2, s2, _ = t2.get_rows(signs)
    assert (w2 == w).all() and (s2[:, :5] == st[:, :5]).all() and (s2.view(np.int32)[:, 5] == 0).all()  # delta_show is not saved


def test_rows_due_for_elimination_are_not_saved():
    t, signs = small(oracle.ADAGRAD, show_threshold=5.0)
    st = np.array([[0.1, 3, 0, 0], [2, 7, 0, 0]], np.float32)
    t.set_rows(signs, np.ones((2, 2), np.float32), st)
    rows = t.serialize_block(0, "txt").decode().split("\n")[2:-2]
    assert len(rows) == 1 and rows[0].startswith("16\t")
