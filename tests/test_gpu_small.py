"""The path of few launches that small batches take (every slot within 4096 lookups, at most 128 slots, at
most 256 k lookups: tensornet_amd/csrc/small_batch.h), through the C ABI against the CPU oracle at the bar of
test_gpu_sparse.py (mapped ids and pulled rows bit for bit, updated rows within 1e-5 / 1e-7): the shapes on
either side of its limits, several workgroups per slot, signs with many records on either side of the
threshold from which a wavefront applies them, inserts, and that a batch of its kind does take it."""
import numpy as np
import pytest
import torch

from tensornet_amd import _lib, synth

from helpers import Pair, all_signs, check_pull, dev

pytestmark = pytest.mark.gpu

ADAGRAD_HP = dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8)
ADAM_HP = dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8)
FTRL_HP = dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0)


def kernels_of(tn, fn):
    """Names of the library's kernels that fn() launches."""
    lib = _lib.load()
    lib.tn_profile_reset()
    lib.tn_profile_enable(1)
    try:
        fn()
        torch.cuda.synchronize()
    finally:
        lib.tn_profile_enable(0)
    names = set(_lib.profile_summary())
    lib.tn_profile_reset()
    return names


def batch(rng, slots, per, pool, hot=0, fresh=None):
    """`slots` slots of `per` lookups from pool (Zipf-like through squaring); the first `hot` signs of the pool
    sit in every slot; `fresh` replaces a share of the lookups by signs nobody has seen."""
    out = []
    for _ in range(slots):
        idx = (rng.random(per) ** 2 * len(pool)).astype(np.int64)
        v = pool[idx].copy()
        if hot:
            v[:hot] = pool[:hot]
        if fresh:
            k = rng.random(per) < fresh
            v[k] = rng.integers(1, 1 << 62, int(k.sum()))
        out.append(v)
    return out


@pytest.mark.parametrize("slots,per,opt,hyper,dim", [
    (1, 1, "AdaGrad", ADAGRAD_HP, 8),          # one lookup
    (3, 4096, "AdaGrad", ADAGRAD_HP, 16),      # the largest slot of the path, eight workgroups per slot
    (3, 4097, "AdaGrad", ADAGRAD_HP, 16),      # one lookup too many: the path of two bucket levels
    (5, 513, "Adam", ADAM_HP, 16),             # two workgroups per slot
    (128, 40, "AdaGrad", ADAGRAD_HP, 8),       # the most slots of the path
    (129, 40, "AdaGrad", ADAGRAD_HP, 8),       # one slot too many
    (12, 300, "Ftrl", FTRL_HP, 4),             # the most slots without k_apply_big: signs with up to 12 records by lane groups
    (13, 300, "Ftrl", FTRL_HP, 4),             # ... with it: 5 records or more by a wavefront
    (26, 1024, "Adam", ADAM_HP, 16),
    (7, 1000, "AdaGrad", ADAGRAD_HP, 6),       # rows that are no multiple of four floats: the scalar update kernels
])
def test_shapes_on_either_side_of_the_limits(tn, oracle, slots, per, opt, hyper, dim):
    rng = np.random.default_rng(slots * 10007 + per)
    pool = synth.splitmix64(np.arange(1, 20001, dtype=np.uint64)).view(np.int64)
    pair = Pair(tn, oracle, opt, dim, hyper, reserve=400000, zero_init=True)  # (new rows: zeros on both sides)
    pair.populate(pool[:5000].view(np.uint64))  # the rest of the pool, and the fresh signs, are inserted by the pulls
    seen = []
    for step in range(3):
        values = batch(rng, slots, per, pool, hot=min(per, 3), fresh=0.05 if step else None)
        counts = check_pull(pair, values)
        grads = synth.make_grads(counts, pair.wf, 0.01, seed=step)
        labels = [(rng.random(len(v)) < 0.3).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        seen.append(all_signs(values))
        assert pair.assert_rows_match(seen[-1]) > 0.99
    check_pull(pair, values)  # the updated rows come back
    pair.assert_rows_match(np.unique(np.concatenate(seen)))


def test_a_small_batch_takes_the_path_of_few_launches(tn, oracle):
    """cfg1's shape (1024 x 8 slots): the pull is three launches and the push two, none of them a kernel of the
    path of two bucket levels; 4097 lookups in a slot, and the other path runs."""
    D = 8
    pool = synth.splitmix64(np.arange(1, 3001, dtype=np.uint64)).view(np.int64)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP)
    pair.populate(pool.view(np.uint64))
    rng = np.random.default_rng(5)

    def step(per):
        values = [dev(v) for v in batch(rng, 8, per, pool)]
        gvars = [torch.zeros((per + 1, D), device="cuda") for _ in values]
        pulled = kernels_of(tn, lambda: tn.ops.sparse_table_pull(gvars, values, pair.h))
        counts = tn.ops.sparse_table_last_unique_counts(pair.h, 8)
        grads = [torch.zeros((c, D), device="cuda") for c in counts]
        labels = [torch.zeros_like(v) for v in values]
        pushed = kernels_of(tn, lambda: tn.ops.sparse_table_push(values, grads, labels, pair.h))
        tn.ops.sparse_table_sync(pair.h)
        return pulled, pushed

    pulled, pushed = step(1024)
    assert pulled == {"k_small_slots", "k_small_group_finish<4>", "k_group_emit<true>"}
    assert len(pushed) == 2 and "k_small_verify<true>" in pushed and any(k.startswith("k_small_apply") for k in pushed)
    pulled, pushed = step(4097)
    assert "k_lds_dedup<true>" in pulled and not any(k.startswith("k_small") for k in pulled | pushed)


def test_a_gradient_matrix_with_too_few_rows_is_reported(tn, oracle):
    """A push on the plan of a small pull whose gradient matrix has fewer rows than its slot has distinct signs:
    TN_ERR_INVALID_ARGUMENT from the push itself; the records that have a gradient row are applied, as on the
    other paths."""
    D = 8
    pool = synth.splitmix64(np.arange(1, 101, dtype=np.uint64)).view(np.int64)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP)
    pair.populate(pool.view(np.uint64))
    values = [pool[:60].copy(), pool[40:100].copy()]
    counts = check_pull(pair, values)
    assert counts.tolist() == [60, 60]
    grads = [np.full((60, D), 0.1, np.float32), np.full((59, D), 0.1, np.float32)]  # slot 1: one row short
    labels = [np.zeros(60, np.int64)] * 2
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.sparse_table_push([dev(v) for v in values], [dev(g) for g in grads], [dev(l) for l in labels], pair.h)
    assert e.value.code == 1
    tn.ops.sparse_table_sync(pair.h)
    # the oracle applies what has a row: slot 0 whole, slot 1 without its last distinct sign
    rc, _ = pair.o.push_op([values[0], values[1][:59]], [grads[0], grads[1]], [labels[0], labels[1][:59]])
    assert rc == 0
    pair.assert_rows_match(all_signs(values))


def test_small_and_large_batches_alternate_on_one_table(tn, oracle):
    """The two paths share the table's plan and scratch buffers: small, large, small, with a push of each, and
    a push of the small batch after the large pull (another batch than the last pull's)."""
    D = 16
    rng = np.random.default_rng(77)
    pool = synth.splitmix64(np.arange(1, 30001, dtype=np.uint64)).view(np.int64)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=300000, zero_init=True)
    pair.populate(pool[:20000].view(np.uint64))
    small = batch(rng, 6, 700, pool, hot=2)
    large = batch(rng, 6, 9000, pool, hot=2)
    seen = []
    for values in (small, large, small, large, small):
        counts = check_pull(pair, values)
        grads = synth.make_grads(counts, D, 0.01, seed=len(seen))
        pair.push_op(values, grads, [np.ones(len(v), np.int64) for v in values])
        seen.append(all_signs(values))
        assert pair.assert_rows_match(seen[-1]) > 0.99
    counts = check_pull(pair, large)
    small_counts = pair.o.pull_op(small, [np.zeros((len(v) + 1, pair.wf), np.float32) for v in small])[2]
    grads = synth.make_grads(small_counts, D, 0.01, seed=9)
    pair.push_op(small, grads, [np.zeros(len(v), np.int64) for v in small])
    pair.assert_rows_match(np.unique(np.concatenate(seen)))


@pytest.mark.parametrize("opt,hyper,dim,slots,per", [("AdaGrad", ADAGRAD_HP, 8, 8, 1024), ("Adam", ADAM_HP, 16, 26, 2000),
                                                     ("Ftrl", FTRL_HP, 4, 40, 500)])
def test_both_paths_leave_the_same_table(tn, oracle, opt, hyper, dim, slots, per):
    """Two tables, the same seed and the same batches, one on the path of few launches and one with it switched off:
    mapped ids, pulled rows (new rows included: same seed, same signs) and the rows after every push are the same
    bit for bit -- both paths apply a sign's records in slot order with the same arithmetic."""
    rng = np.random.default_rng(99)
    pool = synth.splitmix64(np.arange(1, 40001, dtype=np.uint64)).view(np.int64)
    tables = []
    for small in (True, False):
        gopt = getattr(tn.core, opt)(**hyper)
        h = tn.core.create_sparse_table(gopt, "", dim, False, "")
        tn.core.reserve_sparse_table(h, 300000)
        tn.core.set_sparse_table_seed(h, 1234)
        tn.core.set_sparse_table_small_batch_path(h, small)
        tables.append(h)
    wf, sf = tn.core.sparse_table_row_layout(tables[0])
    seen = []
    for step in range(3):
        values = batch(rng, slots, per, pool, hot=3, fresh=0.1)
        gvalues = [dev(v) for v in values]
        labels = [dev((rng.random(len(v)) < 0.3).astype(np.int64)) for v in values]
        outs = []
        for h in tables:
            gvars = [torch.full((per + 1, wf), -7.0, device="cuda") for _ in values]
            launched = kernels_of(tn, lambda: outs.append((tn.ops.sparse_table_pull(gvars, gvalues, h), gvars)))
            assert any(k.startswith("k_small") for k in launched) == (h == tables[0])
        counts = tn.ops.sparse_table_last_unique_counts(tables[0], slots)
        assert counts == tn.ops.sparse_table_last_unique_counts(tables[1], slots)
        for a, b in zip(outs[0][0], outs[1][0]):
            assert torch.equal(a, b)
        for a, b in zip(outs[0][1], outs[1][1]):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32))
        grads = [dev(g) for g in synth.make_grads(counts, wf, 0.01, seed=step)]
        for h in tables:
            tn.ops.sparse_table_push(gvalues, grads, labels, h)
            tn.ops.sparse_table_sync(h)
        seen.append(all_signs(values))
        signs = dev(np.unique(np.concatenate(seen)).view(np.int64))
        w0, s0, f0 = tn.ops.table_export_rows(tables[0], signs)
        w1, s1, f1 = tn.ops.table_export_rows(tables[1], signs)
        assert bool(f0.all()) and bool(f1.all())
        assert torch.equal(w0.view(torch.int32), w1.view(torch.int32))
        assert torch.equal(s0.view(torch.int32), s1.view(torch.int32))
    assert tn.core.sparse_table_key_count(tables[0]) == tn.core.sparse_table_key_count(tables[1])
