"""Seeded random shapes through the pull and push ops against the CPU oracle, at the bar of test_gpu_sparse.py (mapped
ids and pulled rows bit for bit, updated rows within 1e-5 / 1e-7): slot counts on either side of the 128 of the slot
masks, slot lengths on either side of the 4096 of the small-batch path, empty slots, vocabularies from a few dozen
signs (every sign in every slot) to mostly distinct ones, new signs, all three optimizers, the cvm columns."""
import numpy as np
import pytest

from tensornet_amd import synth

from helpers import Pair, all_signs, check_pull

pytestmark = pytest.mark.gpu

HP = {"AdaGrad": dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8),
      "Adam": dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8),
      "Ftrl": dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0)}


@pytest.mark.parametrize("block", range(6))
def test_random_shapes(tn, oracle, block):
    for case in range(10):
        seed = 424200 + block * 10 + case
        rng = np.random.default_rng(seed)
        opt = ["AdaGrad", "Adam", "Ftrl"][int(rng.integers(0, 3))]
        D = int(rng.choice([4, 8, 16, 64, 12]))
        cvm = bool(rng.random() < 0.2) and opt == "AdaGrad"
        N = int(rng.choice([1, 2, 7, 26, 40, 100, 128, 131]))
        maxlen = int(rng.choice([3, 60, 700, 4096, 4097, 9000]))
        maxlen = min(maxlen, 400000 // N)
        vocab = int(rng.choice([50, 3000, 200000]))
        fresh = float(rng.choice([0.0, 0.02, 0.3]))
        what = "seed %d: %s D=%d cvm=%d N=%d maxlen=%d vocab=%d fresh=%.2f" % (seed, opt, D, cvm, N, maxlen, vocab, fresh)
        pair = Pair(tn, oracle, opt, D, HP[opt], use_cvm=cvm, reserve=1500000, zero_init=True, seed=seed)
        pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64) + np.uint64(seed)).view(np.int64)
        pair.populate(pool[: max(1, vocab * 2 // 3)].view(np.uint64))
        seen = []
        try:
            for step in range(3):
                values = []
                for _ in range(N):
                    n = int(rng.integers(0, maxlen + 1)) if rng.random() < 0.9 else 0
                    v = pool[(rng.random(n) ** 2 * vocab).astype(np.int64)]
                    if fresh and n:
                        k = rng.random(n) < fresh
                        v = v.copy()
                        v[k] = rng.integers(1, 1 << 62, int(k.sum()))
                    values.append(v)
                if sum(len(v) for v in values) == 0:
                    continue
                counts = check_pull(pair, values, loose_col=(D + 1) if cvm else None)
                grads = synth.make_grads(counts, pair.wf, 0.01, seed=step)
                labels = [(rng.random(len(v)) < 0.3).astype(np.int64) * int(rng.integers(1, 3)) for v in values]
                pair.push_op(values, grads, labels)
                seen.append(all_signs(values))
                pair.assert_rows_match(seen[-1])
            if seen:
                pair.assert_rows_match(np.unique(np.concatenate(seen)))
        except AssertionError as e:
            raise AssertionError(what + "\n" + str(e))
        tn.core.clear_sparse_table(pair.h)
