"""Seeded random large batches (1.2 to 4.5 M lookups: one stream and several) through pull and push ops queued
back to back, three steps a case: the three optimizers, rows of 4 to 64 elements, 40 to 128 slots whose lengths
differ from step to step (so that every call lays its plan out anew), up to 10 % signs the table has never seen,
detached updates and the exact comparison of the signs switched on and off at random.  Against the CPU oracle
(core/kernels/sparse_table_ops.cc:170-265,317-368): mapped ids bit for bit, pulled rows and the rows after the
pushes within 1e-5 relative / 1e-7 absolute."""
import numpy as np
import pytest
import torch

from tensornet_amd import synth

from helpers import ATOL, RTOL, Pair, all_signs, dev

pytestmark = pytest.mark.gpu

HP = {"AdaGrad": dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8),
      "Adam": dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8),
      "Ftrl": dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0)}


@pytest.mark.parametrize("seed", [3100040, 3100034, 538, 148, 52, 35])
def test_random_large_batches_back_to_back(tn, oracle, seed):
    rng = np.random.default_rng(seed)
    opt = ["AdaGrad", "Adam", "Ftrl"][int(rng.integers(0, 3))]
    D = int(rng.choice([4, 8, 16, 32, 64]))
    N = int(rng.choice([40, 64, 100, 128]))
    total = int(rng.choice([300000, 1200000, 3300000, 4500000]))
    per = total // N
    vocab = int(rng.choice([100000, 600000]))
    fresh = float(rng.choice([0.0, 0.01, 0.1]))
    detached = bool(rng.random() < 0.5)
    exact = bool(rng.random() < 0.3)
    what = "%s D=%d N=%d per=%d vocab=%d fresh=%.2f detached=%d exact=%d" % (opt, D, N, per, vocab, fresh, detached, exact)
    pair = Pair(tn, oracle, opt, D, HP[opt], reserve=3000000, zero_init=True, seed=seed)
    tn.core.set_sparse_table_detached_updates(pair.h, detached)
    tn.core.set_sparse_table_exact_verify(pair.h, exact)
    pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64) + np.uint64(seed)).view(np.int64)
    pair.populate(pool.view(np.uint64))
    steps = []
    for step in range(3):
        values = []
        for s in range(N):
            n = int(per * rng.uniform(0.7, 1.0))
            v = pool[(rng.random(n) ** 3 * vocab).astype(np.int64)]
            if fresh:
                k = rng.random(n) < fresh
                v = v.copy()
                v[k] = rng.integers(1, 1 << 62, int(k.sum()))
            values.append(v)
        counts = [len(np.unique(v)) for v in values]
        steps.append(dict(values=values, gvalues=[dev(v) for v in values],
                          gvars=[torch.zeros((len(v) + 1, D), device="cuda") for v in values],
                          grads=synth.make_grads(counts, D, 0.01, seed=step),
                          labels=[(rng.random(len(v)) < 0.2).astype(np.int64) for v in values]))
    for st in steps:
        st["ggrads"] = [dev(g) for g in st["grads"]]
        st["glabels"] = [dev(l) for l in st["labels"]]
    for st in steps:  # the device side, back to back
        st["gmapped"] = tn.ops.sparse_table_pull(st["gvars"], st["gvalues"], pair.h)
        tn.ops.sparse_table_push(st["gvalues"], st["ggrads"], st["glabels"], pair.h)
    tn.ops.sparse_table_sync(pair.h)
    try:
        seen = []
        for st in steps:
            cvars = [np.zeros((len(v) + 1, D), np.float32) for v in st["values"]]
            rc, cmapped, counts = pair.o.pull_op(st["values"], cvars)
            assert rc == 0
            for s in range(N):
                assert (st["gmapped"][s].cpu().numpy() == cmapped[s]).all(), "mapped ids of slot %d" % s
                np.testing.assert_allclose(st["gvars"][s].cpu().numpy(), cvars[s], rtol=RTOL, atol=ATOL)
            assert pair.o.push_op(st["values"], st["grads"], st["labels"])[0] == 0
            seen.append(all_signs(st["values"]))
        pair.assert_rows_match(np.unique(np.concatenate(seen)))
    except AssertionError as e:
        raise AssertionError(what + "\n" + str(e))
