"""tn_sparse_table_pull_static, the entry point that allocates nothing, against tn_sparse_table_pull:
same outputs bit for bit, on two calls in a row (the second smaller, so that what the first left in
the static scratch array lies beyond it), through the C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

from tensornet_amd import synth

pytestmark = pytest.mark.gpu


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _table(tn, dim, resident, seed):
    opt = tn.core.AdaGrad(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8)
    h = tn.core.create_sparse_table(opt, "", dim, False, "")
    tn.core.reserve_sparse_table(h, 400000)
    tn.core.set_sparse_table_seed(h, seed)
    w = synth.snapshot_rows(resident, dim)
    tn.ops.table_load_rows(h, torch.from_numpy(resident.view(np.int64)).cuda(), torch.from_numpy(w).cuda())
    return h


def test_static_pull_matches_the_allocating_pull(tn):
    from tensornet_amd import _lib

    lib = _lib.load()
    dim = 16
    rng = np.random.default_rng(5)
    pool = synth.splitmix64(np.arange(1, 300001, dtype=np.uint64))
    resident = pool[:100000]
    ha = _table(tn, dim, resident, seed=99)   # driven through tn_sparse_table_pull
    hb = _table(tn, dim, resident, seed=99)   # driven through tn_sparse_table_pull_static
    for n in (120000, 700):  # resident signs, absent signs (inserted and initialised), repeats
        req = pool[rng.integers(0, 300000, n)]
        req[: n // 50] = req[0]
        signs = torch.from_numpy(req.view(np.int64)).cuda()
        out_a = torch.full((n, dim), -3.0, device="cuda")
        out_b = torch.full((n, dim), -5.0, device="cuda")
        _lib.check(lib.tn_sparse_table_pull(ha, _ptr(signs), n, dim, _ptr(out_a), _stream()))
        # the call allocates nothing: the device's free memory is the same before and after (hipMemGetInfo;
        # the tensors above are allocated already, and torch's caching allocator is not called in between)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        _lib.check(lib.tn_sparse_table_pull_static(hb, _ptr(signs), n, dim, _ptr(out_b), _stream()))
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(out_a.view(torch.int32), out_b.view(torch.int32))
        assert tn.core.sparse_table_key_count(ha) == tn.core.sparse_table_key_count(hb)
        # resident rows are the snapshot's, bit for bit
        known = np.isin(req, resident)
        assert known.any() and (~known).any()
        expect = synth.snapshot_rows(req[known], dim)
        assert (out_b.cpu().numpy()[known].view(np.int32) == expect.view(np.int32)).all()
    # the rows the static pulls inserted are in the table: an ordinary pull of them finds the same values
    signs = torch.from_numpy(pool.view(np.int64)).cuda()
    before = tn.core.sparse_table_key_count(hb)
    w_a, _, f_a = tn.ops.table_export_rows(ha, signs)
    w_b, _, f_b = tn.ops.table_export_rows(hb, signs)
    assert torch.equal(f_a, f_b) and torch.equal(w_a.view(torch.int32), w_b.view(torch.int32))
    assert tn.core.sparse_table_key_count(hb) == before


def test_static_pull_refuses_what_it_cannot_do_without_allocating(tn):
    from tensornet_amd import _lib

    lib = _lib.load()
    dim = 8
    fresh = tn.core.create_sparse_table(tn.core.AdaGrad(), "", dim, False, "")
    signs = torch.arange(1, 9, dtype=torch.int64, device="cuda")
    out = torch.zeros((8, dim), device="cuda")
    rc = lib.tn_sparse_table_pull_static(fresh, _ptr(signs), 8, dim, _ptr(out), _stream())
    assert rc == 11 and b"no storage yet" in lib.tn_last_error()
    h = _table(tn, dim, synth.splitmix64(np.arange(1, 101, dtype=np.uint64)), seed=1)
    too_many = (1 << 20) + 1
    rc = lib.tn_sparse_table_pull_static(h, _ptr(signs), too_many, dim, _ptr(out), _stream())
    assert rc == 11 and b"at most 1048576" in lib.tn_last_error()
    rc = lib.tn_sparse_table_pull_static(h, _ptr(signs), 8, dim + 1, _ptr(out), _stream())
    assert rc == 3
    # a small table that would have to grow
    small = tn.core.create_sparse_table(tn.core.AdaGrad(), "", dim, False, "")
    tn.core.reserve_sparse_table(small, 100)
    tn.ops.table_load_rows(small, signs, torch.zeros((8, dim), device="cuda"))
    many = torch.arange(1000, 5000, dtype=torch.int64, device="cuda")
    out2 = torch.zeros((4000, dim), device="cuda")
    rc = lib.tn_sparse_table_pull_static(small, _ptr(many), 4000, dim, _ptr(out2), _stream())
    assert rc == 6 and b"would have to grow" in lib.tn_last_error()
    assert tn.core.sparse_table_key_count(small) == 8
