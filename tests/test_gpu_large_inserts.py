"""Large batches that insert new signs, queued back to back: the path a training loop (and the benchmark)
runs on every step.

A pull of 3 M lookups or more spreads its work over the table's streams: the table is probed per distinct
record beside the grouping and the ranking, every second-level bucket lists the rows it inserted, those rows
are filled by a kernel of their own, and the push's descriptors are staged beside the pull's gather.  Here
three such batches of slightly different sizes -- about 1 % of their lookups signs the table has never seen, then
25 % -- go through bound
pull and push ops with no host wait in between but the ones the calls make themselves, and every output is
compared with the CPU oracle (core/kernels/sparse_table_ops.cc:170-265,317-368,
core/ps/optimizer/optimizer_kernel.h:299-308): mapped ids and the pulled rows of resident signs bit for bit,
the rows after every push within 1e-5 relative / 1e-7 absolute, the number of resident keys exactly.

A new row's initial weights are random draws on both sides, so the oracle is given the row the device drew
(taken from the pulled variable of the very pull that inserted it) before it replays the step; the draws
themselves are held to the initialiser's distribution (mean and standard deviation within 1 %)."""
import numpy as np
import pytest
import torch

from tensornet_amd import synth

from helpers import ATOL, RTOL, Pair, dev

pytestmark = pytest.mark.gpu

D = 16
SCALE = 0.1
HP = dict(learning_rate=0.01, initial_g2sum=0.1, initial_scale=SCALE, epsilon=1e-8)
VOCAB = 400000
SLOTS, PER = 64, 53500  # 3.3-3.4 M lookups: above the size from which a call uses the table's side streams


def make_batches(pool):
    rng = np.random.default_rng(31337)
    hot = pool[:30]
    batches = []
    next_fresh = 10 ** 9
    # (slots a little longer from batch to batch... and shorter again: every call lays its plan out anew)
    for share, per in ((0.01, PER), (0.012, PER - 1500), (0.25, PER - 700)):
        n_fresh = int(share * SLOTS * per / 3)  # every fresh sign about three times, in one slot or in several
        fresh = synth.splitmix64(np.arange(next_fresh, next_fresh + n_fresh, dtype=np.uint64)).view(np.int64)
        next_fresh += n_fresh
        values = []
        for _ in range(SLOTS):
            v = pool[(rng.random(per) ** 3 * VOCAB).astype(np.int64)]
            take = rng.random(per) < share
            v[take] = fresh[rng.integers(0, n_fresh, int(take.sum()))]
            v[: len(hot)] = hot  # signs with a record in every slot
            values.append(v)
        batches.append(values)
    # the second batch again at the end: every sign resident by now, the rows those of two pushes ago
    batches.append(batches[1])
    return batches


@pytest.mark.parametrize("detached,exact", [(False, False), (True, False), (True, True)])
def test_large_batches_with_new_signs_back_to_back(tn, oracle, detached, exact):
    pair = Pair(tn, oracle, "AdaGrad", D, HP, reserve=3 * 10 ** 6, seed=5)
    tn.core.set_sparse_table_detached_updates(pair.h, detached)
    # (with the exact comparison of the signs a pull also writes its copy of them, behind the plan's group arrays)
    tn.core.set_sparse_table_exact_verify(pair.h, exact)
    base = pair.populate(synth.splitmix64(np.arange(1, VOCAB + 1, dtype=np.uint64)))
    pool = base.view(np.int64)
    batches = make_batches(pool)
    assert all(sum(len(v) for v in b) >= 3 << 20 for b in batches)
    steps = []
    for k, values in enumerate(batches):
        counts = [len(np.unique(v)) for v in values]
        rng = np.random.default_rng(100 + k)
        st = dict(values=values, gvalues=[dev(v) for v in values],
                  gvars=[torch.full((len(v) + 1, D), -7.0, device="cuda") for v in values],
                  grads=synth.make_grads(counts, D, 0.01, seed=k),
                  labels=[(rng.random(len(v)) < 0.2).astype(np.int64) for v in values])
        st["ggrads"] = [dev(g) for g in st["grads"]]
        st["glabels"] = [dev(l) for l in st["labels"]]
        st["pull"] = tn.ops.BoundSparseTablePull(st["gvars"], st["gvalues"], pair.h)
        st["push"] = tn.ops.BoundSparseTablePush(st["gvalues"], st["ggrads"], st["glabels"], pair.h)
        steps.append(st)
    # the device side: every call queued as soon as the one before has returned
    for st in steps:
        st["gmapped"] = [m.clone() for m in st["pull"]()]
        st["push"]()
    tn.ops.sparse_table_sync(pair.h)
    gpu_keys = tn.core.sparse_table_key_count(pair.h)

    # the oracle, call by call
    sigma = SCALE / np.sqrt(D)
    seen = [base]
    total_new = 0
    for k, st in enumerate(steps):
        values = st["values"]
        gm = [m.cpu().numpy() for m in st["gmapped"]]
        gv = [v.cpu().numpy() for v in st["gvars"]]
        cat = np.concatenate(values).view(np.uint64)
        signs, first = np.unique(cat, return_index=True)
        _, _, found = pair.o.get_rows(signs)
        unseen = ~found.astype(bool)
        # the row the device drew for every sign it inserted: wherever the sign occurs it reads that one row
        offs = np.cumsum([0] + [len(v) for v in values])
        slot_of = np.searchsorted(offs, first[unseen], side="right") - 1
        new_rows = np.stack([gv[s][gm[s][p - offs[s]]] for s, p in zip(slot_of, first[unseen])]) if unseen.any() \
            else np.zeros((0, D), np.float32)
        if k < 3:
            assert unseen.sum() > 0.002 * len(cat)
            assert abs(new_rows.mean()) < 0.01 * sigma, "mean of the new rows"
            assert abs(new_rows.std() / sigma - 1) < 0.01, "standard deviation of the new rows"
        else:
            assert not unseen.any()
        total_new += int(unseen.sum())
        pair.o.set_rows(signs[unseen], new_rows)
        cvars = [np.full((len(v) + 1, D), -7.0, np.float32) for v in values]
        rc, cmapped, counts = pair.o.pull_op(values, cvars)
        assert rc == 0
        exact = 0
        for s in range(SLOTS):
            assert (gm[s] == cmapped[s]).all(), "mapped ids of slot %d, step %d" % (s, k)
            if k == 0:  # nothing pushed yet: snapshot rows, new rows and the untouched tail bit for bit
                assert (gv[s].view(np.int32) == cvars[s].view(np.int32)).all(), "rows of slot %d" % s
            else:
                np.testing.assert_allclose(gv[s], cvars[s], rtol=RTOL, atol=ATOL)
            exact += int((gv[s].view(np.int32) == cvars[s].view(np.int32)).all(axis=1).sum())
        assert exact > 0.99 * sum(len(c) for c in cvars)
        assert pair.o.push_op(values, st["grads"], st["labels"])[0] == 0
        seen.append(signs)
    assert gpu_keys == VOCAB + total_new == pair.o.key_count()
    assert pair.assert_rows_match(np.unique(np.concatenate(seen))) > 0.99
