"""GPU parity of ShowDecay / DeleteByShow against the oracle, through the C ABI
(state compared bit for bit: one float multiply per field)."""
import numpy as np
import pytest
import torch

from tensornet_amd import synth

from helpers import Pair, dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("opt,dim,hyper", [
    ("AdaGrad", 16, dict(learning_rate=0.01, initial_g2sum=0.1, show_decay_rate=0.9, show_threshold=2.5, no_show_days=3)),
    ("AdaGrad", 6, dict(learning_rate=0.01, initial_g2sum=0.1, show_decay_rate=0.7, show_threshold=2.5, no_show_days=3,
                        elimination_logic=1)),
    ("Ftrl", 8, dict(learning_rate=0.05, show_decay_rate=0.8, show_threshold=1.5)),
    ("Adam", 8, dict(learning_rate=1e-3, show_decay_rate=0.5)),
])
def test_show_decay_and_delete_by_show(tn, oracle, opt, dim, hyper):
    rng = np.random.default_rng(dim)
    pair = Pair(tn, oracle, opt, dim, hyper)
    signs = synth.splitmix64(np.arange(1, 3001, dtype=np.uint64))
    signs = np.concatenate([signs, np.array([0, 2 ** 64 - 1], np.uint64)])  # the two extreme signs as well
    base = pair.populate(signs)
    # a few pushes so that show / click / delta_show differ between rows
    for step in range(3):
        values = [base[rng.integers(0, len(base), 700)].view(np.int64) for _ in range(3)]
        pair.pull_op(values)
        counts = [len(np.unique(v)) for v in values]
        grads = synth.make_grads(counts, pair.wf, 0.01, seed=step)
        pair.push_op(values, grads, [rng.integers(0, 2, len(v)).astype(np.int64) for v in values])
    probe = np.concatenate([base, synth.splitmix64(np.arange(10 ** 6, 10 ** 6 + 50, dtype=np.uint64))])
    for delta in (1, 2, 4):
        pair.o.show_decay(delta)
        tn.core.show_decay(pair.h, delta)
        pair.assert_rows_match(base, exact=True)
        got = tn.ops.table_delete_by_show(pair.h, dev(probe.view(np.int64))).cpu().numpy().astype(bool)
        want = pair.o.delete_by_show(probe)
        assert (got == want).all()
    assert want.any() == (opt != "Adam")   # after 7 days some rows are due for elimination (never with Adam)


def test_show_decay_full_table_properties(tn, oracle):
    """2e7 resident rows: every resident row decays exactly once, nothing else changes."""
    dim = 16
    opt = tn.core.AdaGrad(learning_rate=0.01, initial_g2sum=0.1, show_decay_rate=0.5, show_threshold=0.75)
    h = tn.core.create_sparse_table(opt, "", dim, False, "")
    n = 2 * 10 ** 7
    tn.core.reserve_sparse_table(h, n)
    ids = torch.arange(1, n + 1, dtype=torch.int64, device="cuda")
    signs = synth.splitmix64_torch(ids)
    state = torch.zeros((n, 4), device="cuda")
    state[:, 1] = (ids % 7 + 1).float()      # show 1..7
    state[:, 2] = (ids % 3).float()          # click
    tn.ops.table_load_rows(h, signs, synth.snapshot_rows_torch(signs, dim), state)
    sample = signs[:: 997].contiguous()
    w0, s0, f0 = tn.ops.table_export_rows(h, sample)
    tn.core.show_decay(h, 3)
    tn.core.show_decay(h, 4)
    w1, s1, f1 = tn.ops.table_export_rows(h, sample)
    assert bool(f0.all()) and bool(f1.all()) and tn.core.sparse_table_key_count(h) == n
    assert torch.equal(w0, w1) and torch.equal(s0[:, 0], s1[:, 0])
    assert torch.equal(s1[:, 1], s0[:, 1] * 0.25) and torch.equal(s1[:, 2], s0[:, 2] * 0.25)
    assert (s1[:, 3].view(torch.int32) == 7).all()
    flags = tn.ops.table_delete_by_show(h, sample).bool()
    assert torch.equal(flags, s1[:, 1] < 0.75)   # days 7 <= 1000, so only the show test can fire
