"""Signs with many records -- one in most slots of the batch -- on the large-batch path, where a wavefront
owns each of them: AdaGrad rows of every power-of-two dim from 4 to 64 (k_apply_big_adagrad<D>: its chunk is 64
records for dims up to 16, 16 for 32 and 64, so 70 records are several chunks, the last one partial), a dim with
its own general kernel (12), Adam; with the two cvm columns; all against the CPU oracle, record by record in slot
order (core/kernels/sparse_table_ops.cc:336-367, core/ps/table/sparse_table.cc:68-83,
core/ps/optimizer/ada_grad_kernel.cc:105-129): rows within 1e-5 relative / 1e-7 absolute, more than 99 % of them
bit for bit."""
import numpy as np
import pytest

from tensornet_amd import synth

from helpers import Pair, all_signs, check_pull

pytestmark = pytest.mark.gpu

ADAGRAD_HP = dict(learning_rate=0.05, initial_g2sum=0.1, initial_scale=0.1, epsilon=1e-8)
ADAM_HP = dict(learning_rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-8, initial_scale=0.1)
SLOTS = 70


def batch(rng, pool, step):
    """70 slots of 600-900 lookups: 3 signs in every slot (70 records), 5 in the first 40 slots, 6 in 17, 6 in 16,
    6 in 15 (just below the threshold) and a tail of ordinary signs, some of them new in the second step."""
    values = []
    for s in range(SLOTS):
        n = int(rng.integers(600, 900))
        v = pool[rng.integers(100, 20000 if step == 0 else 26000, n)]
        hot = [pool[0:3]]
        if s < 40:
            hot.append(pool[3:8])
        if s < 17:
            hot.append(pool[8:14])
        if s < 16:
            hot.append(pool[14:20])
        if s < 15:
            hot.append(pool[20:26])
        hot = np.concatenate(hot)
        # every hot sign a few times, at random places
        at = rng.choice(n, size=3 * len(hot), replace=False)
        v[at] = np.tile(hot, 3)
        values.append(v)
    return values


@pytest.mark.parametrize("opt,hyper,dim,cvm", [
    ("AdaGrad", ADAGRAD_HP, 4, False), ("AdaGrad", ADAGRAD_HP, 8, True), ("AdaGrad", ADAGRAD_HP, 16, False),
    ("AdaGrad", ADAGRAD_HP, 32, False), ("AdaGrad", ADAGRAD_HP, 64, True), ("AdaGrad", ADAGRAD_HP, 12, False),
    ("Adam", ADAM_HP, 16, False),
])
def test_signs_in_most_slots_on_the_large_batch_path(tn, oracle, opt, hyper, dim, cvm):
    rng = np.random.default_rng(1000 + dim)
    pair = Pair(tn, oracle, opt, dim, hyper, use_cvm=cvm, reserve=200000, zero_init=True)
    tn.core.set_sparse_table_small_batch_path(pair.h, False)  # (slots this short would take the path of few launches)
    pool = synth.splitmix64(np.arange(1, 26001, dtype=np.uint64)).view(np.int64)
    pair.populate(pool[:20000].view(np.uint64))
    for step in range(3):
        values = batch(rng, pool, min(step, 1))
        counts = check_pull(pair, values, loose_col=(dim + 1) if cvm else None)
        grads = synth.make_grads(counts, pair.wf, 0.05, seed=step)
        labels = [(rng.random(len(v)) < 0.3).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        # (with cvm a tenth or so of the columns is the logarithm column, which follows the libm in use)
        assert pair.assert_rows_match(all_signs(values)) > (0.9 if cvm else 0.99)
