"""Dense table checkpoints (DenseTable::Save / Load, core/ps/table/dense_table.cc:103-157)
on the GPU path against the CPU oracle's stream: same text structure, values within the
update tolerance, files readable by either side, training continues after a load."""
import os

import numpy as np
import pytest
import torch

from helpers import ATOL, RTOL, dev

pytestmark = pytest.mark.gpu


def make(tn, oracle, kind):
    if kind == "adam":
        hp = dict(beta1=0.9, beta2=0.999, epsilon=1e-8)
        return tn.core.create_dense_table(tn.core.Adam(learning_rate=1e-3, **hp)), (oracle.ADAM, hp)
    hp = dict(initial_g2sum=0.5, epsilon=1e-3, grad_decay_rate=0.9, mom_decay_rate=0.5)
    return tn.core.create_dense_table(tn.core.AdaGrad(**hp)), (oracle.ADAGRAD, hp)


def dense_file(path, handle):
    return os.path.join(str(path), "dense_table", str(handle), "0")


def tokens(text):
    """Header tokens as strings, numbers as floats, line structure kept."""
    out = []
    for line in text.split("\n"):
        if ":" in line:
            k, v = line.split(":")
            out.append((k, v if k == "opt_name" else float(v)))
        else:
            out.append(tuple(float(x) for x in line.split("\t")) if line else ())
    return out


@pytest.mark.parametrize("kind", ["adam", "adagrad"])
def test_save_matches_oracle_and_load_continues(tn, oracle, kind, tmp_path):
    total = 1003  # blocks of 126, last one 121
    rng = np.random.default_rng(len(kind))
    h, (okind, hp) = make(tn, oracle, kind)
    d = oracle.Dense(okind, total, **hp)
    w0 = rng.uniform(-0.05, 0.05, total).astype(np.float32)
    d.set_weight(w0)
    var = dev(w0)
    tn.ops.dense_table_init([var], h)
    for _ in range(3):
        g = (rng.standard_normal(total) * 1e-2).astype(np.float32)
        d.apply(g, 0.01)
        tn.ops.dense_table_push_pull([var], [dev(g)], 0.01, h)
    tn.core.save_dense_table(h, tmp_path)
    got = open(dense_file(tmp_path, h)).read()
    want = d.serialize().decode()
    tg, tw = tokens(got), tokens(want)
    assert len(tg) == len(tw)
    for a, b in zip(tg, tw):
        assert len(a) == len(b)
        if a and isinstance(a[0], str):
            assert a[0] == b[0]
            if a[0] == "opt_name":
                assert a[1] == b[1]
            else:
                assert a[1] == pytest.approx(b[1], rel=2e-6)
        elif a:
            np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-7)  # 6 printed digits of values within RTOL
    # the file the GPU path wrote loads into the oracle, and the oracle's into a new table
    d2 = oracle.Dense(okind, total, **hp)
    d2.deserialize(got.encode())
    d.save(str(tmp_path / "o"), 7)
    h2, _ = make(tn, oracle, kind)
    os.makedirs(os.path.dirname(dense_file(tmp_path / "o", h2)), exist_ok=True)
    os.replace(dense_file(tmp_path / "o", 7), dense_file(tmp_path / "o", h2))
    tn.core.load_dense_table(h2, tmp_path / "o")  # initialises the table from the file
    d3 = oracle.Dense(okind, total, **hp)
    d3.load(str(tmp_path / "o"), h2)
    np.testing.assert_array_equal(tn.ops.dense_table_get_weight(h2).cpu().numpy(), d3.get_weight())
    states = tn.ops.dense_table_get_state(h2, 2 if kind == "adam" else 3)
    for i, s in enumerate(states):
        np.testing.assert_array_equal(s.cpu().numpy(), d3.get_state(i))
    # one more step on both: the beta powers came back too
    g = (rng.standard_normal(total) * 1e-2).astype(np.float32)
    var2 = torch.zeros(total, device="cuda")
    d3.apply(g, 0.01)
    tn.ops.dense_table_push_pull([var2], [dev(g)], 0.01, h2)
    np.testing.assert_allclose(var2.cpu().numpy(), d3.get_weight(), rtol=RTOL, atol=ATOL)
    # saving the loaded table gives the oracle's file back byte for byte
    h3, _ = make(tn, oracle, kind)
    os.makedirs(os.path.dirname(dense_file(tmp_path / "o", h3)), exist_ok=True)
    with open(dense_file(tmp_path / "o", h3), "wb") as f:
        f.write(want.encode())
    tn.core.load_dense_table(h3, tmp_path / "o")
    tn.core.save_dense_table(h3, tmp_path / "again")
    assert open(dense_file(tmp_path / "again", h3)).read() == want


def test_dense_checkpoint_errors(tn, oracle, tmp_path):
    h, _ = make(tn, oracle, "adam")
    tn.core.save_dense_table(h, tmp_path)  # never initialised: nothing is written (dense_table.cc:106-109)
    assert not os.path.exists(dense_file(tmp_path, h))
    with pytest.raises(tn.TensorNetError):
        tn.core.load_dense_table(h, tmp_path)  # no file
    tn.ops.dense_table_init([torch.zeros(16, device="cuda")], h)
    tn.core.save_dense_table(h, tmp_path)
    text = open(dense_file(tmp_path, h)).read()

    def put(handle, body):
        os.makedirs(os.path.dirname(dense_file(tmp_path, handle)), exist_ok=True)
        with open(dense_file(tmp_path, handle), "w") as f:
            f.write(body)

    big, _ = make(tn, oracle, "adam")
    tn.ops.dense_table_init([torch.zeros(17, device="cuda")], big)
    put(big, text)
    with pytest.raises(tn.TensorNetError) as e:  # CHECK in DenseTable::Init, dense_table.cc:38-44
        tn.core.load_dense_table(big, tmp_path)
    assert e.value.code == 8
    other, _ = make(tn, oracle, "adagrad")
    put(other, text)
    with pytest.raises(tn.TensorNetError, match="last trained model with optimizer is:Adam"):
        tn.core.load_dense_table(other, tmp_path)
    shards, _ = make(tn, oracle, "adam")
    put(shards, text.replace("rank_num:1", "rank_num:2"))
    with pytest.raises(tn.TensorNetError, match="shards"):
        tn.core.load_dense_table(shards, tmp_path)
    cut, _ = make(tn, oracle, "adam")
    put(cut, text[: len(text) // 2])
    with pytest.raises(tn.TensorNetError, match="malformed"):
        tn.core.load_dense_table(cut, tmp_path)


@pytest.mark.parametrize("kind", ["adam", "adagrad"])
@pytest.mark.parametrize("total,shards", [(1003, 3), (10, 4), (5, 8)])
def test_shards_of_one_table(tn, oracle, kind, total, shards, tmp_path):
    """A table cut into shards (DenseTable::Init, dense_table.cc:46-66): every shard updates
    its own range of the variables, all shards together equal the unsharded oracle table,
    and each writes its own checkpoint file."""
    rng = np.random.default_rng(total * shards)
    every = -(-total // shards)
    w0 = rng.uniform(-0.05, 0.05, total).astype(np.float32)
    sizes = [total // 3, total - total // 3]  # two variables; the shard borders cut through them
    cuts = [(0, sizes[0]), (sizes[0], total)]
    _, (okind, hp) = make(tn, oracle, kind)
    whole = oracle.Dense(okind, total, **hp)
    whole.set_weight(w0)
    tables, ranges = [], []
    for r in range(shards):
        opt = tn.core.Adam(learning_rate=1e-3, **hp) if kind == "adam" else tn.core.AdaGrad(**hp)
        h = tn.core.create_dense_table(opt, shards, r)
        tn.ops.dense_table_init([dev(w0[a:b]) for a, b in cuts], h)
        b, e = tn.ops.dense_table_range(h)
        assert (b, e) == (min(r * every, total), min((r + 1) * every, total))
        tables.append(h)
        ranges.append((b, e))
    merged = w0.copy()
    for step in range(3):
        g = (rng.standard_normal(total) * 1e-2).astype(np.float32)
        whole.apply(g, 0.01)
        for h, (b, e) in zip(tables, ranges):
            vars_ = [torch.full((n,), 7.0, device="cuda") for n in sizes]
            tn.ops.dense_table_push_pull(vars_, [dev(g[a:c]) for a, c in cuts], 0.01, h)
            got = torch.cat(vars_).cpu().numpy()
            outside = np.ones(total, bool)
            outside[b:e] = False
            assert (got[outside] == 7.0).all()  # other shards' ranges are not this worker's to write
            merged[b:e] = got[b:e]
    np.testing.assert_allclose(merged, whole.get_weight(), rtol=RTOL, atol=ATOL)
    for r, (h, (b, e)) in enumerate(zip(tables, ranges)):
        np.testing.assert_array_equal(tn.ops.dense_table_get_weight(h).cpu().numpy(), merged[b:e])
        tn.core.save_dense_table(h, tmp_path)
        path = os.path.join(str(tmp_path), "dense_table", str(h), str(r))
        if e == b:
            assert not os.path.exists(path)  # a shard past the end has no kernel and writes nothing
            continue
        text = open(path).read()
        assert text.startswith("total_elements:%d\nrank_num:%d\n" % (total, shards))
        part = oracle.Dense(okind, e - b, **hp)
        part.deserialize(text.encode(), shard_num=shards, table_total=total)
        np.testing.assert_array_equal(part.get_weight(), np.array([float("%g" % x) for x in merged[b:e]], np.float32))
        # a fresh shard table takes the file back
        opt = tn.core.Adam(learning_rate=1e-3, **hp) if kind == "adam" else tn.core.AdaGrad(**hp)
        h2 = tn.core.create_dense_table(opt, shards, r)
        os.makedirs(os.path.join(str(tmp_path), "dense_table", str(h2)), exist_ok=True)
        with open(os.path.join(str(tmp_path), "dense_table", str(h2), str(r)), "w") as f:
            f.write(text)
        tn.core.load_dense_table(h2, tmp_path)
        assert tn.ops.dense_table_range(h2) == (b, e)
        np.testing.assert_array_equal(tn.ops.dense_table_get_weight(h2).cpu().numpy(), part.get_weight())
