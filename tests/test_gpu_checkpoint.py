"""Save / load of the sparse table in the reference's checkpoint formats: the files the
HIP side writes hold exactly the records the oracle writes (same bytes per record; the
order of rows inside a file is not defined in the reference either), and each side loads the
other's files."""
import gzip
import os

import numpy as np
import pytest
import torch

from tensornet_amd import synth
from tensornet_amd._lib import TensorNetError

from helpers import Pair, dev

pytestmark = pytest.mark.gpu

CASES = [
    ("AdaGrad", 16, False, dict(learning_rate=0.01, initial_g2sum=0.1, show_threshold=0.5)),
    ("AdaGrad", 6, True, dict(learning_rate=0.01, initial_g2sum=0.1)),
    ("Adam", 8, False, dict(learning_rate=1e-3)),
    ("Ftrl", 4, False, dict(learning_rate=0.05, show_threshold=0.5)),
]


def trained_pair(tn, oracle, opt, dim, use_cvm, hyper, rows=5000):
    rng = np.random.default_rng(dim)
    pair = Pair(tn, oracle, opt, dim, hyper, use_cvm=use_cvm)
    signs = synth.splitmix64(np.arange(1, rows + 1, dtype=np.uint64))
    signs = np.concatenate([signs, np.array([0, 2 ** 64 - 1], np.uint64)])
    base = pair.populate(signs)
    for step in range(2):   # some rows get state, the others stay at show 0 (and may be due for elimination)
        values = [base[rng.integers(0, len(base), 900)].view(np.int64) for _ in range(3)]
        pair.pull_op(values)
        counts = [len(np.unique(v)) for v in values]
        grads = synth.make_grads(counts, pair.wf, 0.01, seed=step)
        pair.push_op(values, grads, [rng.integers(0, 2, len(v)).astype(np.int64) for v in values])
    return pair, base


def records(path, mode, record_bytes):
    data = gzip.open(path, "rb").read()
    if mode == "txt":
        lines = data.decode().split("\n")
        assert lines[-2:] == ["", ""]
        return lines[:2], sorted(lines[2:-2])
    assert data[-1:] == b"\n" and (len(data) - 5) % record_bytes == 0
    body = data[4:-1]
    return data[:4], sorted(body[i:i + record_bytes] for i in range(0, len(body), record_bytes))


@pytest.mark.parametrize("opt,dim,use_cvm,hyper", CASES)
@pytest.mark.parametrize("mode", ["txt", "bin"])
def test_saved_files_match_the_oracle_and_load_both_ways(tn, oracle, tmp_path, opt, dim, use_cvm, hyper, mode):
    pair, base = trained_pair(tn, oracle, opt, dim, use_cvm, hyper)
    gdir, cdir = str(tmp_path / "gpu"), str(tmp_path / "cpu")
    tn.core.save_sparse_table(pair.h, gdir, mode)
    pair.o.save(cdir, pair.h, mode)
    value = dim * 4 + 12 + (4 if use_cvm else 0) if opt == "AdaGrad" else 3 * dim * 4 + 4
    total = 0
    for b in range(8):
        sub = os.path.join("sparse_table", str(pair.h), "rank_0", "block_%d.gz" % b)
        ghead, grec = records(os.path.join(gdir, sub), mode, 8 + value)
        chead, crec = records(os.path.join(cdir, sub), mode, 8 + value)
        assert ghead == chead and grec == crec
        total += len(grec)
    kept = int((~pair.o.delete_by_show(base)).sum())
    assert total == kept and (kept < len(base)) == ("show_threshold" in hyper)
    # a name without suffix is read as text by the reference: give binary files the _bin suffix
    suffix = "_bin" if mode == "bin" else ""
    if suffix:
        for d in (gdir, cdir):
            r = os.path.join(d, "sparse_table", str(pair.h), "rank_0")
            for b in range(8):
                os.rename(os.path.join(r, "block_%d.gz" % b), os.path.join(r, "block_%d_bin.gz" % b))
    # the oracle loads the GPU's files, a fresh GPU table loads the oracle's
    o2 = oracle.Table(pair.o.kind if hasattr(pair.o, "kind") else {"AdaGrad": 0, "Adam": 1, "Ftrl": 2}[opt], dim,
                      use_cvm=use_cvm, buckets=1 << 12, **hyper)
    assert o2.load(gdir, pair.h, mode, suffix=suffix) == kept
    h2 = tn.core.create_sparse_table(pair.gopt, "", dim, use_cvm, "")
    os.rename(os.path.join(cdir, "sparse_table", str(pair.h)), os.path.join(cdir, "sparse_table", str(h2)))
    tn.core.load_sparse_table(h2, cdir, "txt")     # the mode comes from the file names
    assert tn.core.sparse_table_key_count(h2) == kept
    gw, gs, gf = tn.ops.table_export_rows(h2, dev(base.view(np.int64)))
    cw, cs, cf = o2.get_rows(base)
    assert (gf.cpu().numpy() == cf).all() and int(cf.sum()) == kept
    sel = cf.astype(bool)
    assert (gw.cpu().numpy()[sel].view(np.int32) == cw[sel].view(np.int32)).all()
    assert (gs.cpu().numpy()[sel].view(np.int32) == cs[sel].view(np.int32)).all()
    if mode == "bin":   # the binary format keeps every saved field exactly (not saved: delta_show, click without cvm)
        w0, s0, _ = pair.o.get_rows(base)
        cols = ([0, 1, 3] + ([2] if use_cvm else [])) if opt == "AdaGrad" else list(range(2 * dim + 1))
        assert (cw[sel][:, :dim] == w0[sel][:, :dim]).all()
        assert (cs[sel][:, cols].view(np.int32) == s0[sel][:, cols].view(np.int32)).all()


def test_named_table_directory_and_errors(tn, oracle, tmp_path):
    opt = tn.core.AdaGrad(learning_rate=0.01)
    h = tn.core.create_sparse_table(opt, "user_embedding", 4, False, "")
    signs = synth.splitmix64_torch(torch.arange(1, 101, dtype=torch.int64, device="cuda"))
    tn.ops.table_load_rows(h, signs, torch.ones((100, 4), device="cuda"))
    tn.core.save_sparse_table(h, str(tmp_path), "bin")
    d = tmp_path / "sparse_table" / "user_embedding" / "rank_0"
    assert sorted(os.listdir(d)) == ["block_%d.gz" % b for b in range(8)]
    adam = tn.core.create_sparse_table(tn.core.Adam(learning_rate=0.01), "user_embedding", 4, False, "")
    tn.core.save_sparse_table(h, str(tmp_path), "txt")
    with pytest.raises(TensorNetError):     # saved with another optimizer
        tn.core.load_sparse_table(adam, str(tmp_path), "txt")
    with pytest.raises(TensorNetError):     # nothing there
        tn.core.load_sparse_table(h, str(tmp_path / "missing"), "txt")


def test_two_million_rows_round_trip(tn, oracle, tmp_path):
    """Several export / load rounds (the table is read out 2^20 slots at a time, rows go back in
    batches of 2^20): every row comes back bit for bit from the binary format."""
    import time

    dim, n = 16, 2 * 10 ** 6
    opt = tn.core.AdaGrad(learning_rate=0.01, initial_g2sum=0.1)
    h = tn.core.create_sparse_table(opt, "big", dim, False, "")
    tn.core.reserve_sparse_table(h, n)
    ids = torch.arange(1, n + 1, dtype=torch.int64, device="cuda")
    signs = synth.splitmix64_torch(ids)
    state = torch.zeros((n, 4), device="cuda")
    state[:, 0] = 0.1 + (ids % 5).float()
    state[:, 1] = (ids % 7).float()
    state[:, 3] = (ids % 11).int().view(torch.float32)
    tn.ops.table_load_rows(h, signs, synth.snapshot_rows_torch(signs, dim), state)
    t0 = time.time()
    tn.core.save_sparse_table(h, str(tmp_path), "bin")
    t1 = time.time()
    r = tmp_path / "sparse_table" / "big" / "rank_0"
    for b in range(8):
        os.rename(r / ("block_%d.gz" % b), r / ("block_%d_bin.gz" % b))
    h2 = tn.core.create_sparse_table(opt, "big", dim, False, "")
    tn.core.load_sparse_table(h2, str(tmp_path), "bin")
    t2 = time.time()
    print("save %.1f s, load %.1f s for %d rows" % (t1 - t0, t2 - t1, n))
    assert tn.core.sparse_table_key_count(h2) == n
    sample = signs[::101].contiguous()
    w0, s0, f0 = tn.ops.table_export_rows(h, sample)
    w1, s1, f1 = tn.ops.table_export_rows(h2, sample)
    assert bool(f1.all()) and torch.equal(w0, w1)
    assert torch.equal(s0[:, [0, 1, 3]].view(torch.int32), s1[:, [0, 1, 3]].view(torch.int32))
