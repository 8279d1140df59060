"""GPU parity of the combiner around the pull / push ops (forward:
embedding_lookup_sparse on the pulled rows; backward: push fed with pooled
gradients, reduced per distinct sign on the device) against oracle/combine.py
and the table oracle, through the C ABI.  Tolerance 1e-5 relative / 1e-7
absolute (sums run in the same order on both sides; the scale factors may
differ in the last bit)."""
import numpy as np
import pytest
import torch

from oracle import combine as C
from tensornet_amd import synth
from tensornet_amd._lib import TensorNetError

from helpers import ATOL, RTOL, Pair, all_signs, dev

pytestmark = pytest.mark.gpu

ADAGRAD_HP = dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8)
ADAM_HP = dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8)
NAMES = {C.SUM: "sum", C.MEAN: "mean", C.SQRTN: "sqrtn"}


def ragged_slots(rng, slots, batch, vocab, mean_len):
    """Per slot: signs and the example of every lookup (sorted), some slots empty, some examples empty."""
    pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)).view(np.int64)
    values, examples = [], []
    for s in range(slots):
        if s % 4 == 3:
            n = np.zeros(batch, np.int64)
        else:
            n = rng.poisson(mean_len, batch)
        ex = np.repeat(np.arange(batch, dtype=np.int64), n)
        values.append(pool[rng.integers(0, vocab, len(ex))])
        examples.append(ex)
    return values, examples


@pytest.mark.parametrize("dim,combiner", [(16, C.MEAN), (16, C.SUM), (16, C.SQRTN), (6, C.MEAN)])
def test_forward_and_pooled_push_against_the_oracle(tn, oracle, dim, combiner):
    rng = np.random.default_rng(5 + dim + combiner)
    batch, slots, vocab = 300, 7, 900
    pair = Pair(tn, oracle, "AdaGrad", dim, ADAGRAD_HP)
    pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)), seed=3)
    for step in range(2):
        values, examples = ragged_slots(rng, slots, batch, vocab, 2.5)
        gm, gv, cm, cv, counts = pair.pull_op(values)
        gex = [dev(e) for e in examples]
        out = tn.ops.embedding_lookup_sparse(gv, gm, gex, batch, pair.h, NAMES[combiner])
        for s in range(slots):
            want = C.combine_forward(cm[s], examples[s], cv[s], batch, combiner)
            np.testing.assert_allclose(out[s].cpu().numpy(), want, rtol=RTOL, atol=ATOL)
        pooled = [rng.standard_normal((batch, dim)).astype(np.float32) * 0.01 for _ in range(slots)]
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        grads = [C.combine_backward(cm[s], examples[s], pooled[s], batch, combiner, int(counts[s]))
                 for s in range(slots)]
        assert pair.o.push_op(values, grads, labels)[0] == 0
        tn.ops.sparse_table_push_pooled([dev(v) for v in values], gex, [dev(p) for p in pooled],
                                        [dev(l) for l in labels], pair.h, NAMES[combiner])
        tn.ops.sparse_table_sync(pair.h)
        assert pair.assert_rows_match(all_signs(values)) > 0.9


def test_pooled_push_of_another_batch_than_the_last_pull(tn, oracle):
    """No pull before the push: the push analyses the batch itself, then reduces and applies."""
    rng = np.random.default_rng(2)
    batch, slots, vocab, dim = 200, 5, 600, 8
    pair = Pair(tn, oracle, "Adam", dim, ADAM_HP)
    pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    values, examples = ragged_slots(rng, slots, batch, vocab, 3.0)
    rc, cm, counts = pair.o.pull_op(values, [np.zeros((len(v) + 1, dim), np.float32) for v in values])
    pooled = [rng.standard_normal((batch, dim)).astype(np.float32) * 0.01 for _ in range(slots)]
    labels = [np.zeros(len(v), np.int64) for v in values]
    grads = [C.combine_backward(cm[s], examples[s], pooled[s], batch, C.MEAN, int(counts[s])) for s in range(slots)]
    assert pair.o.push_op(values, grads, labels)[0] == 0
    tn.ops.sparse_table_push_pooled([dev(v) for v in values], [dev(e) for e in examples], [dev(p) for p in pooled],
                                    [dev(l) for l in labels], pair.h, "mean")
    tn.ops.sparse_table_sync(pair.h)
    pair.assert_rows_match(all_signs(values))


def test_combine_rejects_bad_example_ids_and_ids(tn, oracle):
    pair = Pair(tn, oracle, "AdaGrad", 4, ADAGRAD_HP)
    var = [torch.zeros((5, 4), device="cuda")]
    ids = [dev(np.array([0, 1, 2], np.int64))]
    with pytest.raises(TensorNetError):  # not sorted
        tn.ops.embedding_lookup_sparse(var, ids, [dev(np.array([1, 0, 2], np.int64))], 3, pair.h)
    with pytest.raises(TensorNetError):  # beyond the batch
        tn.ops.embedding_lookup_sparse(var, ids, [dev(np.array([0, 1, 3], np.int64))], 3, pair.h)
    with pytest.raises(TensorNetError):  # id beyond the variable
        tn.ops.embedding_lookup_sparse(var, [dev(np.array([0, 1, 7], np.int64))], [dev(np.array([0, 1, 2], np.int64))],
                                       3, pair.h)
    out = tn.ops.embedding_lookup_sparse(var, ids, [dev(np.array([0, 1, 2], np.int64))], 3, pair.h)
    assert float(out[0].abs().sum()) == 0.0


def test_pooled_push_with_unsorted_example_ids_changes_nothing(tn, oracle):
    """Example ids that are not sorted (or lie outside the batch) cannot be reduced: the push is
    reported as failed at the next synchronising call and leaves every row as it was."""
    rng = np.random.default_rng(4)
    batch, slots, vocab, dim = 100, 3, 300, 8
    pair = Pair(tn, oracle, "AdaGrad", dim, ADAGRAD_HP)
    base = pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    values, examples = ragged_slots(rng, slots, batch, vocab, 3.0)
    pair.pull_op(values)
    pooled = [dev(rng.standard_normal((batch, dim)).astype(np.float32)) for _ in range(slots)]
    labels = [dev(np.zeros(len(v), np.int64)) for v in values]
    for spoil in ("unsorted", "out of range"):
        bad = [e.copy() for e in examples]
        if spoil == "unsorted":
            bad[1][[0, -1]] = bad[1][[-1, 0]]
        else:
            bad[0][-1] = batch
        tn.ops.sparse_table_push_pooled([dev(v) for v in values], [dev(e) for e in bad], pooled, labels, pair.h, "mean")
        with pytest.raises(TensorNetError):
            tn.ops.sparse_table_sync(pair.h)
        pair.assert_rows_match(base, exact=True)


def test_full_size_pooled_push_equals_push_of_reduced_gradients(tn, oracle):
    """cfg3-sized batch (16384 x 100 slots, ~5 M lookups): a pooled push must leave the table in
    the state a plain push leaves it in when the per-distinct-sign gradients are reduced by torch
    (index_add of the scaled example rows), and the forward pass must satisfy the adjoint identity
    with that reduction."""
    cfg = synth.CONFIGS["cfg3"]
    dim, batch = cfg["dim"], cfg["batch"]
    values_np = synth.make_batch(cfg, 1)
    rng = np.random.default_rng(0)
    examples = []
    for v in values_np:  # spread the slot's lookups over the examples, sorted
        examples.append(np.sort(rng.integers(0, batch, len(v))).astype(np.int64))
    tables = []
    for k in range(2):
        opt = tn.core.AdaGrad(**cfg["hyper"])
        h = tn.core.create_sparse_table(opt, "", dim, False, "")
        tn.core.reserve_sparse_table(h, 4 * 10 ** 6)
        tn.core.set_sparse_table_seed(h, 5)
        tables.append(h)
    gvalues = [dev(v) for v in values_np]
    gex = [dev(e) for e in examples]
    labels = [torch.zeros_like(v) for v in gvalues]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    pooled = [torch.randn((batch, dim), device="cuda", generator=gen) * 0.01 for _ in gvalues]
    outs = []
    for h in tables:
        gvars = [torch.zeros((len(v) + 1, dim), device="cuda") for v in values_np]
        mapped = tn.ops.sparse_table_pull(gvars, gvalues, h)   # both tables insert the same rows (same seed)
        outs.append((gvars, mapped))
    gvars, mapped = outs[0]
    fwd = tn.ops.embedding_lookup_sparse(gvars, mapped, gex, batch, tables[0], "mean")
    reduced, lhs, rhs = [], 0.0, 0.0
    for s in range(len(gvalues)):
        cnt = torch.bincount(gex[s], minlength=batch).clamp(min=1).to(torch.float32)
        per_lookup = pooled[s][gex[s]] / cnt[gex[s]][:, None]
        g = torch.zeros_like(gvars[s]).index_add_(0, mapped[s], per_lookup)
        reduced.append(g)
        lhs += float((fwd[s].double() * pooled[s].double()).sum())
        rhs += float((gvars[s].double() * g.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))
    tn.ops.sparse_table_push_pooled(gvalues, gex, pooled, labels, tables[0], "mean")
    tn.ops.sparse_table_push(gvalues, reduced, labels, tables[1])
    tn.ops.sparse_table_sync(tables[0])
    tn.ops.sparse_table_sync(tables[1])
    signs = torch.unique(torch.cat(gvalues))
    w0, s0, f0 = tn.ops.table_export_rows(tables[0], signs)
    w1, s1, f1 = tn.ops.table_export_rows(tables[1], signs)
    assert bool(f0.all()) and bool(f1.all())
    torch.testing.assert_close(w0, w1, rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(s0[:, :3], s1[:, :3], rtol=1e-4, atol=1e-6)
