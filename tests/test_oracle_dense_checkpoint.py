"""The oracle's dense checkpoint stream against the format the reference writes
(core/ps/table/dense_table.cc:103-157, optimizer_kernel.h:139-160,224-235,
adam_kernel.cc:57-87, ada_grad_kernel.cc:50-76).  The reference holds no file of
this kind, so the expected texts below are written out by hand from those
stream operators; floats print as operator<< prints them (6 significant digits)."""
import numpy as np
import pytest

import oracle.cpu as oracle


def test_adam_text_by_hand():
    d = oracle.Dense(oracle.ADAM, 3)  # ceil(3 / 8) = 1 element per block: 3 blocks
    d.set_weight(np.array([0.5, -1.25, 1e-7], np.float32))
    block = "opt_name:Adam\narray_size:1\nbeta1_power:1\nbeta2_power:1\n%s\t0\t0\n\n\n"
    expect = "total_elements:3\nrank_num:1\n" + block % "0.5" + block % "-1.25" + block % "1e-07"
    assert d.serialize().decode() == expect


def test_adagrad_text_by_hand():
    d = oracle.Dense(oracle.ADAGRAD, 10, initial_g2sum=0.1)  # ceil(10 / 8) = 2: 5 blocks
    d.set_weight(np.arange(10, dtype=np.float32) / 4)
    text = d.serialize().decode()
    expect = "total_elements:10\nrank_num:1\n"
    for b in range(5):
        expect += "opt_name:AdaGrad\narray_size:2\n"
        for i in (2 * b, 2 * b + 1):
            expect += "%g\t0\t0.1\t0\n" % (i / 4)
        expect += "\n\n"
    assert text == expect


def test_last_block_is_short():
    d = oracle.Dense(oracle.ADAM, 1003)  # blocks of 126, the last holds 1003 - 7 * 126 = 121
    sizes = [int(l.split(":")[1]) for l in d.serialize().decode().split("\n") if l.startswith("array_size:")]
    assert sizes == [126] * 7 + [121]


@pytest.mark.parametrize("kind", [oracle.ADAM, oracle.ADAGRAD])
def test_round_trip_keeps_six_digits(kind):
    total = 77
    rng = np.random.default_rng(kind)
    a = oracle.Dense(kind, total)
    a.set_weight(rng.uniform(-1, 1, total).astype(np.float32))
    for _ in range(3):
        a.apply(rng.standard_normal(total).astype(np.float32), 0.01)
    text = a.serialize()
    b = oracle.Dense(kind, total)
    b.deserialize(text)
    # what a reader of the text gets: every float rounded to 6 significant digits
    for got, want in [(b.get_weight(), a.get_weight())] + [(b.get_state(i), a.get_state(i)) for i in range(3)]:
        np.testing.assert_array_equal(got, np.array([float("%g" % x) for x in want], np.float32))
    if kind == oracle.ADAM:
        p1, p2 = a.beta_powers()
        assert p1 == pytest.approx(0.9 ** 3, rel=1e-6) and p2 == pytest.approx(0.999 ** 3, rel=1e-6)
        for blk in range(b.num_blocks()):
            assert b.beta_powers(blk) == (np.float32("%g" % p1), np.float32("%g" % p2))
    assert b.serialize() == text  # printing 6 digits of a 6-digit value changes nothing


def test_mismatches_are_refused():
    text = oracle.Dense(oracle.ADAM, 16).serialize()
    with pytest.raises(ValueError, match="total"):
        oracle.Dense(oracle.ADAM, 17).deserialize(text)
    with pytest.raises(ValueError, match="optimizer"):
        oracle.Dense(oracle.ADAGRAD, 16).deserialize(text)
    with pytest.raises(ValueError, match="shard"):
        oracle.Dense(oracle.ADAM, 16).deserialize(text, shard_num=2)


def test_shard_file_header_names_the_whole_table():
    # shard 1 of 3 over 10 elements holds [4, 8): ceil(10 / 3) = 4 per shard (dense_table.cc:46-60)
    d = oracle.Dense(oracle.ADAGRAD, 4)
    text = d.serialize(rank_num=3, table_total=10).decode()
    assert text.startswith("total_elements:10\nrank_num:3\nopt_name:AdaGrad\narray_size:1\n")
    assert text.count("array_size:1\n") == 4  # ceil(4 / 8) = 1 element per block
    oracle.Dense(oracle.ADAGRAD, 4).deserialize(text.encode(), shard_num=3, table_total=10)
