"""GPU parity of the sparse pull / push path against the CPU oracle, through
the C ABI.  Bar: mapped ids and pulled rows bit-exact; post-update weights and
state within 1e-5 relative / 1e-7 absolute; integer state exact."""
import numpy as np
import pytest
import torch

from tensornet_amd import synth

from helpers import ATOL, RTOL, Pair, all_signs, check_pull, dev

pytestmark = pytest.mark.gpu

ADAGRAD_HP = dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8)
ADAM_HP = dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8)
FTRL_HP = dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0)


def random_batch(rng, slots, max_len, vocab, ragged=True):
    pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)).view(np.int64)
    out = []
    for _ in range(slots):
        n = int(rng.integers(0, max_len + 1)) if ragged else max_len
        out.append(pool[rng.integers(0, vocab, n)])
    return out


def test_cfg1_pull_then_push(tn, oracle):
    """The reference's own CPU-runnable case: 1024 x 8 single-id slots, dim 8 AdaGrad."""
    cfg = synth.CONFIGS["cfg1"]
    pair = Pair(tn, oracle, "AdaGrad", cfg["dim"], cfg["hyper"], reserve=1 << 20)
    values = synth.make_batch(cfg, 0)
    assert sum(len(v) for v in values) == 8192
    # resident set: every key of the 1e6 vocabulary that the batch can touch is loaded on both sides
    resident = synth.splitmix64(np.arange(1, 200001, dtype=np.uint64))
    pair.populate(np.concatenate([resident, all_signs(values)]))
    counts = check_pull(pair, values)
    grads = synth.make_grads(counts, cfg["dim"], cfg["grad_sigma"])
    labels = [np.zeros(len(v), np.int64) for v in values]
    pair.push_op(values, grads, labels)
    same = pair.assert_rows_match(all_signs(values))
    assert same > 0.99
    check_pull(pair, values)  # pulling again returns the updated rows


@pytest.mark.parametrize("opt,dim,hyper", [
    ("AdaGrad", 16, ADAGRAD_HP), ("AdaGrad", 64, ADAGRAD_HP), ("AdaGrad", 1, ADAGRAD_HP), ("AdaGrad", 6, ADAGRAD_HP),
    ("Adam", 16, ADAM_HP), ("Adam", 8, ADAM_HP), ("Adam", 3, ADAM_HP),
    ("Ftrl", 1, FTRL_HP), ("Ftrl", 16, FTRL_HP),
])
def test_multi_batch_parity(tn, oracle, opt, dim, hyper):
    """Several ragged batches with labels; the same sign occurs in several slots."""
    rng = np.random.default_rng(dim * 7 + len(opt))
    pair = Pair(tn, oracle, opt, dim, hyper)
    vocab = 3000
    pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)), seed=dim)
    touched = []
    sigma = 0.6 if opt == "Ftrl" else 0.01
    for b in range(4):
        values = random_batch(rng, 7, 900, vocab)
        if b == 1:
            values[3] = values[3][:0]  # an empty slot in the middle
        counts = check_pull(pair, values)
        grads = [(rng.standard_normal((int(u), dim)) * sigma).astype(np.float32) for u in counts]
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        touched.append(all_signs(values))
        pair.assert_rows_match(np.unique(np.concatenate(touched)))
    assert tn.core.sparse_table_key_count(pair.h) == pair.o.key_count()


def test_cvm_columns(tn, oracle):
    rng = np.random.default_rng(5)
    pair = Pair(tn, oracle, "AdaGrad", 8, ADAGRAD_HP, use_cvm=True)
    assert pair.wf == 10
    pair.populate(synth.splitmix64(np.arange(1, 501, dtype=np.uint64)))
    for _ in range(2):
        values = random_batch(rng, 3, 400, 500)
        counts = check_pull(pair, values, loose_col=9)
        grads = [(rng.standard_normal((int(u), 10)) * 0.01).astype(np.float32) for u in counts]
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        pair.assert_rows_match(all_signs(values))


def test_extreme_signs_and_single_lookups(tn, oracle):
    """Signs 0, 2^63 and 2^64-1 (the hash table's own free marker) are ordinary keys."""
    pair = Pair(tn, oracle, "AdaGrad", 4, ADAGRAD_HP)
    special = np.asarray([0, 1 << 63, (1 << 64) - 1, 1], dtype=np.uint64)
    pair.populate(special)
    values = [special.view(np.int64)[[2, 0, 2, 1, 3, 2]], special.view(np.int64)[[2]], special.view(np.int64)[[0, 0]]]
    counts = check_pull(pair, values)
    assert counts.tolist() == [4, 1, 1]
    grads = [np.full((int(u), 4), 0.5 + i, np.float32) for i, u in enumerate(counts)]
    labels = [np.ones(len(v), np.int64) for v in values]
    pair.push_op(values, grads, labels)
    pair.assert_rows_match(special)
    (gw, gs, gf), _ = pair.export(special)
    assert gs[2, 1] == 4.0 and gs[2, 2] == 4.0  # sign 2^64-1: show = 3 + 1, click likewise


def test_same_sign_in_many_slots_is_sequential(tn, oracle):
    """A sign present in k slots gets k Applies, slot 0 first -- not one Apply of the sum."""
    D, k = 16, 37
    pair = Pair(tn, oracle, "AdaGrad", D, dict(learning_rate=0.1, initial_g2sum=0.1, epsilon=1e-8))
    hot = synth.splitmix64(np.asarray([42], dtype=np.uint64))
    others = synth.splitmix64(np.arange(100, 100 + k, dtype=np.uint64))
    pair.populate(np.concatenate([hot, others]))
    values = [np.asarray([others[s], hot[0], others[s], hot[0]], dtype=np.uint64).view(np.int64) for s in range(k)]
    counts = check_pull(pair, values)
    rng = np.random.default_rng(0)
    grads = [(rng.standard_normal((int(u), D)) * 0.3).astype(np.float32) for u in counts]
    labels = [np.zeros(len(v), np.int64) for v in values]
    pair.push_op(values, grads, labels)
    pair.assert_rows_match(np.concatenate([hot, others]))
    # the summed-gradient shortcut would give a visibly different row
    ref = oracle.Table(oracle.ADAGRAD, D, buckets=64, learning_rate=0.1, initial_g2sum=0.1, epsilon=1e-8)
    ref.set_rows(hot, synth.snapshot_rows(hot, D))
    info = np.zeros(1, dtype=oracle.sign_info_dtype)
    info["sign"], info["batch_show"] = hot[0], 2 * k
    ref.push(info, sum(g[1] for g in grads)[None, :])
    (gw, _, _), _ = pair.export(hot)
    assert np.abs(gw - ref.get_rows(hot)[0]).max() > 1e-3


def test_new_keys_are_inserted_and_initialised(tn, oracle):
    """Pull of unseen signs inserts rows drawn from N(0, scale/sqrt(D)) (mean / std
    within 1 %), deterministic in (seed, sign); they then behave like any row."""
    D, scale = 16, 0.1
    hp = dict(learning_rate=0.01, initial_g2sum=0.1, initial_scale=scale, epsilon=1e-8)
    pair = Pair(tn, oracle, "AdaGrad", D, hp, reserve=400000, seed=3)
    fresh = synth.splitmix64(np.arange(10 ** 6, 10 ** 6 + 60000, dtype=np.uint64))
    values = [fresh[:40000].view(np.int64), fresh[30000:].view(np.int64)]
    gvars = [torch.zeros((len(v) + 1, D), device="cuda") for v in values]
    gm = tn.ops.sparse_table_pull(gvars, [dev(v) for v in values], pair.h)
    assert tn.core.sparse_table_key_count(pair.h) == 60000
    assert (gm[0].cpu().numpy() == np.arange(40000)).all()
    w = torch.cat([gvars[0][:40000], gvars[1][10000:30000]]).cpu().numpy()
    sigma = scale / np.sqrt(D)
    assert abs(w.mean()) < 0.01 * sigma
    assert abs(w.std() / sigma - 1) < 0.01
    # the same sign pulled through two slots of one call reads one row
    assert torch.equal(gvars[0][30000:40000], gvars[1][:10000])
    (gw, gs, gf), _ = pair.export(fresh)
    assert gf.all() and (gs[:, 0] == np.float32(0.1)).all() and (gs[:, 1:] == 0).all()
    # deterministic: a second table with the same seed draws the same rows
    twin = Pair(tn, oracle, "AdaGrad", D, hp, reserve=400000, seed=3)
    assert torch.equal(tn.ops.table_pull(twin.h, dev(fresh[:1000].view(np.int64)), D), dev(gw[:1000]))
    # continue on both sides from the GPU's rows
    pair.o.set_rows(fresh, gw, gs)
    counts = check_pull(pair, values)
    grads = synth.make_grads(counts, D, 0.01)
    pair.push_op(values, grads, [np.zeros(len(v), np.int64) for v in values])
    pair.assert_rows_match(fresh)
    # Adam / Ftrl rows start with zero moments
    for opt, hyper in (("Adam", ADAM_HP), ("Ftrl", FTRL_HP)):
        p2 = Pair(tn, oracle, opt, 8, dict(hyper, initial_scale=1.0))
        out = tn.ops.table_pull(p2.h, dev(fresh[:20000].view(np.int64)), 8).cpu().numpy()
        assert abs(out.std() * np.sqrt(8) - 1) < 0.01 and abs(out.mean()) < 0.01
        (_, s2, f2), _ = p2.export(fresh[:50])
        assert f2.all() and (s2 == 0).all()
    # sparse_zero_init: rows of zeros
    pz = Pair(tn, oracle, "AdaGrad", 8, ADAGRAD_HP, zero_init=True)
    assert (tn.ops.table_pull(pz.h, dev(fresh[:100].view(np.int64)), 8) == 0).all()


def test_table_level_pull_push_with_repeated_records(tn, oracle):
    """SparseTable::Pull / Push: request order kept; records applied in array order."""
    D = 8
    rng = np.random.default_rng(9)
    for opt, hyper in (("AdaGrad", ADAGRAD_HP), ("Adam", ADAM_HP), ("Ftrl", FTRL_HP)):
        pair = Pair(tn, oracle, opt, D, hyper)
        base = pair.populate(synth.splitmix64(np.arange(1, 301, dtype=np.uint64)))
        req = base[rng.integers(0, 300, 1000)]
        out = tn.ops.table_pull(pair.h, dev(req.view(np.int64)), D).cpu().numpy()
        assert (out.view(np.int32) == pair.o.pull(req).view(np.int32)).all()
        infos = np.zeros(1000, dtype=oracle.sign_info_dtype)
        infos["sign"] = req
        infos["batch_show"] = rng.integers(1, 5, 1000)
        infos["batch_click"] = rng.integers(0, 2, 1000)
        grads = (rng.standard_normal((1000, D)) * (0.5 if opt == "Ftrl" else 0.01)).astype(np.float32)
        assert pair.o.push(infos, grads) == 0
        rec = tn.ops.make_sign_infos(dev(req.view(np.int64)), dev(infos["batch_show"].astype(np.int64)),
                                     dev(infos["batch_click"].astype(np.int64)))
        tn.ops.table_push(pair.h, rec, dev(grads))
        tn.ops.sparse_table_sync(pair.h)
        pair.assert_rows_match(base)


def test_hand_computed_known_answers_on_the_device(tn, oracle):
    """The exact known answers of tests/golden/optim_kat.json (hand-computed from the reference's update rules,
    power-of-two operands, both Ftrl branches and the case that tells float abs from an integer abs) through
    the device path: load the row, push one record, read the row back -- bit for bit."""
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "optim_kat.json")) as f:
        kat = json.load(f)
    sign = np.asarray([0x1234567890ABCDEF], dtype=np.uint64)

    def i2f(i):
        return float(np.asarray([i], dtype=np.int32).view(np.float32)[0])

    def run(opt, dim, hyper, w0, st0, grad, show, click=0):
        h = tn.core.create_sparse_table(getattr(tn.core, opt)(**hyper), "", dim, False, "")
        tn.core.reserve_sparse_table(h, 64)
        tn.ops.table_load_rows(h, dev(sign.view(np.int64)), dev(np.asarray([w0], np.float32)),
                               dev(np.asarray([st0], np.float32)))
        rec = tn.ops.make_sign_infos(dev(sign.view(np.int64)), dev(np.asarray([show], np.int64)),
                                     dev(np.asarray([click], np.int64)))
        tn.ops.table_push(h, rec, dev(np.asarray([grad], np.float32)))
        tn.ops.sparse_table_sync(h)
        w, st, found = tn.ops.table_export_rows(h, dev(sign.view(np.int64)))
        assert int(found[0]) == 1
        return w[0].cpu().numpy(), st[0].cpu().numpy()

    for c in kat["adagrad"]:
        w, st = run("AdaGrad", c["dim"], c["hyper"], c["w0"], c["state0"][:3] + [i2f(c["state0"][3])], c["grad"],
                    c["show"], c["click"])
        assert w.tolist() == c["w1"] and st[:3].tolist() == c["state1"][:3]
        assert int(st[3:4].view(np.int32)[0]) == c["state1"][3]
    for c in kat["adam"]:
        D = c["dim"]
        w, st = run("Adam", D, c["hyper"], c["w0"], c["m0"] + c["v0"] + [0.0, i2f(0)], c["grad"], c["show"])
        assert w.tolist() == c["w1"] and st[:D].tolist() == c["m1"] and st[D:2 * D].tolist() == c["v1"]
        assert int(st[2 * D + 1:2 * D + 2].view(np.int32)[0]) == c["delta_show1"]
    for c in kat["ftrl"]:
        D = c["dim"]
        w, st = run("Ftrl", D, c["hyper"], c["w0"], c["z0"] + c["n0"] + [0.0, i2f(0)], c["grad"], c["show"])
        assert w.tolist() == c["w1"], c["_why"]
        assert st[:D].tolist() == c["z1"] and st[D:2 * D].tolist() == c["n1"]
        assert int(st[2 * D + 1:2 * D + 2].view(np.int32)[0]) == c["delta_show1"]


def test_errors_come_back_as_codes(tn, oracle):
    D = 8
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP)
    signs = pair.populate(synth.splitmix64(np.arange(1, 11, dtype=np.uint64)))
    v = [dev(signs.view(np.int64))]
    # U_s must be strictly smaller than the variable's rows (sparse_table_ops.cc:136)
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.sparse_table_pull([torch.zeros((10, D), device="cuda")], v, pair.h)
    assert e.value.code == 4
    tn.ops.sparse_table_pull([torch.zeros((11, D), device="cuda")], v, pair.h)
    # dim mismatch
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.sparse_table_pull([torch.zeros((11, D + 1), device="cuda")], v, pair.h)
    assert e.value.code == 3
    # push of a sign that was never pulled (optimizer_kernel.h:315): reported, others applied
    unknown = np.asarray([123456789], dtype=np.int64)
    vals = [np.concatenate([signs.view(np.int64)[:3], unknown])]
    tn.ops.sparse_table_push([dev(vals[0])], [torch.full((4, D), 0.1, device="cuda")],
                             [torch.zeros(4, dtype=torch.int64, device="cuda")], pair.h)
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.sparse_table_sync(pair.h)
    assert e.value.code == 5
    pair.o.push_op([vals[0][:3]], [np.full((3, D), 0.1, np.float32)], [np.zeros(3, np.int64)])
    pair.assert_rows_match(signs)
    # bad handle
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.sparse_table_pull([torch.zeros((11, D), device="cuda")], v, 10 ** 6)
    assert e.value.code == 2
    # wrong argument kinds are rejected on the host side
    with pytest.raises(ValueError):
        tn.ops.sparse_table_pull([torch.zeros((11, D))], v, pair.h)
    with pytest.raises(ValueError):
        tn.ops.sparse_table_pull([torch.zeros((11 * D,), device="cuda")], v, pair.h)


def test_table_grows_past_its_reservation(tn, oracle):
    """Load factor 0.75 triggers re-insertion into a larger table (optimizer_kernel.h:266)."""
    D = 4
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=1000)
    cap0 = None
    signs = synth.splitmix64(np.arange(1, 50001, dtype=np.uint64))
    for lo in range(0, 50000, 5000):
        pair.populate(signs[lo:lo + 5000], seed=1)
        cap = tn.core.sparse_table_capacity(pair.h)
        cap0 = cap0 or cap
    assert tn.core.sparse_table_capacity(pair.h) > cap0
    assert tn.core.sparse_table_key_count(pair.h) == 50000
    assert tn.core.sparse_table_key_count(pair.h) <= 0.75 * tn.core.sparse_table_capacity(pair.h)
    pair.assert_rows_match(signs, exact=True)
    # pulls of fresh signs also grow the table
    fresh = synth.splitmix64(np.arange(10 ** 7, 10 ** 7 + 200000, dtype=np.uint64))
    tn.ops.table_pull(pair.h, dev(fresh.view(np.int64)), D)
    assert tn.core.sparse_table_key_count(pair.h) == 250000
    pair.assert_rows_match(signs, exact=True)


def test_cfg2_shape_adam_batches(tn, oracle):
    """Wide&deep-shaped Adam steps (26 single-hot slots, dim 16), resident set scaled
    down, some keys new in every batch; state compared after every batch."""
    cfg = dict(synth.CONFIGS["cfg2"], vocab=2 * 10 ** 5, batch=2048)
    pair = Pair(tn, oracle, "Adam", 16, cfg["hyper"], reserve=1 << 20)
    pair.populate(synth.splitmix64(np.arange(1, 10 ** 5 + 1, dtype=np.uint64)))
    seen = []
    for b in range(6):
        values = synth.make_batch(cfg, b)
        # new keys: let the GPU insert, then mirror its rows into the oracle
        gv = [torch.zeros((len(v) + 1, 16), device="cuda") for v in values]
        tn.ops.sparse_table_pull(gv, [dev(v) for v in values], pair.h)
        signs = all_signs(values)
        (gw, gs, gf), (_, _, cf) = pair.export(signs)
        new = ~cf.astype(bool)
        assert gf.all()
        if b > 0:
            assert 0 < new.mean() < 0.2
        pair.o.set_rows(signs[new], gw[new], gs[new])
        counts = check_pull(pair, values)
        grads = synth.make_grads(counts, 16, cfg["grad_sigma"], seed=b)
        pair.push_op(values, grads, [np.zeros(len(v), np.int64) for v in values])
        seen.append(signs)
        pair.assert_rows_match(np.unique(np.concatenate(seen)))


def test_cfg4_shape_two_tables_same_signs(tn, oracle):
    """Insert-heavy mix: dim-1 Ftrl wide weights and dim-64 AdaGrad embeddings share
    the batch's signs, 20 % of which are fresh."""
    cfg = dict(synth.CONFIGS["cfg4"], vocab=10 ** 5, batch=1024)
    wide = Pair(tn, oracle, "Ftrl", 1, dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0), reserve=1 << 19)
    deep = Pair(tn, oracle, "AdaGrad", 64, dict(learning_rate=0.01, initial_g2sum=0.1), reserve=1 << 19)
    resident = synth.splitmix64(np.arange(1, 10 ** 5 + 1, dtype=np.uint64))
    for pair in (wide, deep):
        pair.populate(resident)
    for b in range(2):
        values = synth.make_batch(cfg, b)
        signs = all_signs(values)
        for pair, sigma in ((wide, 0.5), (deep, 1e-2)):
            gv = [torch.zeros((len(v) + 1, pair.wf), device="cuda") for v in values]
            tn.ops.sparse_table_pull(gv, [dev(v) for v in values], pair.h)
            (gw, gs, gf), (_, _, cf) = pair.export(signs)
            new = ~cf.astype(bool)
            assert 0.1 < new.mean() < 0.7  # 20 % of lookups, a larger share of the distinct signs
            pair.o.set_rows(signs[new], gw[new], gs[new])
            counts = check_pull(pair, values)
            grads = synth.make_grads(counts, pair.wf, sigma, seed=b)
            pair.push_op(values, grads, [np.zeros(len(v), np.int64) for v in values])
            pair.assert_rows_match(signs)


def test_full_size_batch_properties(tn, oracle):
    """cfg3's full batch (16384 x 100 slots, ~5 M lookups) cannot go through the CPU
    oracle in seconds; check size-independent properties instead, on the GPU:
    ids of equal signs agree, ids are dense and in first-occurrence order, the
    variable row of every lookup is the row of its sign, pull is idempotent, and a
    push changes exactly the pulled rows."""
    cfg = synth.CONFIGS["cfg3"]
    D = cfg["dim"]
    opt = tn.core.AdaGrad(**cfg["hyper"])
    h = tn.core.create_sparse_table(opt, "", D, False, "")
    tn.core.reserve_sparse_table(h, 6 * 10 ** 6)
    values = synth.make_batch(cfg, 0)
    L = sum(len(v) for v in values)
    assert 4.5e6 < L < 5.5e6
    gvalues = [dev(v) for v in values]
    uniq = torch.unique(torch.cat(gvalues))
    w0 = synth.snapshot_rows_torch(uniq, D)
    tn.ops.table_load_rows(h, uniq, w0)
    assert tn.core.sparse_table_key_count(h) == uniq.numel()
    rows = [len(v) + 1 for v in values]
    gvars = [torch.full((r, D), 9.0, device="cuda") for r in rows]
    mapped = tn.ops.sparse_table_pull(gvars, gvalues, h)
    counts = tn.ops.sparse_table_last_unique_counts(h, len(values))
    for s in (0, 1, 17, 50, 99):
        v, m = gvalues[s], mapped[s]
        u, inv = torch.unique(v, return_inverse=True)
        assert counts[s] == u.numel() == int(m.max()) + 1
        # first-occurrence order: position of first occurrence increases with the id
        first = torch.full((u.numel(),), len(v), dtype=torch.int64, device="cuda")
        first.scatter_reduce_(0, inv, torch.arange(len(v), device="cuda"), reduce="amin")
        first_by_id = torch.empty_like(first)
        first_by_id[m[first]] = first
        assert bool((first_by_id[1:] > first_by_id[:-1]).all())
        assert torch.equal(m, m[first][inv])  # equal signs <=> equal ids
        # the row a lookup maps to is its sign's snapshot row
        assert torch.equal(gvars[s][m], synth.snapshot_rows_torch(v, D))
        assert bool((gvars[s][counts[s]:] == 9.0).all())
    # idempotent
    gvars2 = [torch.full((r, D), 9.0, device="cuda") for r in rows]
    mapped2 = tn.ops.sparse_table_pull(gvars2, gvalues, h)
    assert all(torch.equal(a, b) for a, b in zip(mapped, mapped2))
    assert all(torch.equal(a, b) for a, b in zip(gvars, gvars2))
    # push with zero gradients: weights unchanged, show counts add up to L
    grads = [torch.zeros((c, D), device="cuda") for c in counts]
    labels = [torch.zeros_like(v) for v in gvalues]
    tn.ops.sparse_table_push(gvalues, grads, labels, h)
    tn.ops.sparse_table_sync(h)
    w1, st1, found = tn.ops.table_export_rows(h, uniq)
    assert bool(found.all()) and torch.equal(w1, w0)
    assert float(st1[:, 1].sum()) == float(L) and bool((st1[:, 0] == 0.1).all())
    # push with a constant gradient g: a key present in k slots gets k sequential Applies,
    # each adding g^2 to g2sum and moving every weight by -lr*g/sqrt(g2sum)
    g = 0.5
    grads = [torch.full((c, D), g, device="cuda") for c in counts]
    tn.ops.sparse_table_push(gvalues, grads, labels, h)
    tn.ops.sparse_table_sync(h)
    w2, st2, _ = tn.ops.table_export_rows(h, uniq)
    k = torch.zeros(uniq.numel(), device="cuda")
    for v in gvalues:
        k[torch.searchsorted(uniq, torch.unique(v))] += 1
    assert float(k.sum()) == float(sum(counts))
    np.testing.assert_allclose(st2[:, 0].cpu().numpy(), (0.1 + k * g * g).cpu().numpy(), rtol=1e-5)
    kmax = int(k.max())
    steps = torch.arange(1, kmax + 1, device="cuda", dtype=torch.float64)
    cum = torch.cumsum(0.01 * g / torch.sqrt(0.1 + steps * g * g), 0)
    expect = w0.double() - cum[(k - 1).long()][:, None]
    np.testing.assert_allclose(w2.cpu().numpy(), expect.cpu().numpy(), rtol=RTOL, atol=1e-6)


def test_push_of_another_batch_than_the_last_pull(tn, oracle):
    """A push reuses what the last pull worked out about its batch only if the
    signs are the same; same-shaped batches with other signs, pushes after
    another table call, and pushes with no pull before them all take the full path."""
    D = 16
    rng = np.random.default_rng(21)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP)
    vocab = 2000
    base = pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    a = random_batch(rng, 5, 700, vocab, ragged=False)
    b = random_batch(rng, 5, 700, vocab, ragged=False)  # same lengths, other signs

    def push(values, seed):
        counts = [len(np.unique(v)) for v in values]
        grads = synth.make_grads(counts, D, 0.01, seed=seed)
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)

    push(a, 0)                      # no pull at all before the first push
    pair.assert_rows_match(base)
    check_pull(pair, a)
    push(b, 1)                      # pull(a) then push(b)
    pair.assert_rows_match(base)
    check_pull(pair, b)
    push(b, 2)                      # the matching push
    push(b, 3)                      # and once more from the same analysis
    pair.assert_rows_match(base)
    check_pull(pair, a)
    tn.ops.table_pull(pair.h, dev(base[:10].view(np.int64)), D)  # a table-level call in between
    b2 = [v.copy() for v in a]
    b2[2][5] = b[2][5]              # one sign differs
    pair.o.pull_op(b2, [np.zeros((len(v) + 1, D), np.float32) for v in b2])
    push(b2, 4)
    pair.assert_rows_match(base)


@pytest.mark.parametrize("slots,opt,hyper", [(40, "AdaGrad", ADAGRAD_HP), (128, "Adam", ADAM_HP),
                                             (130, "AdaGrad", ADAGRAD_HP)])
def test_large_ragged_batches_take_the_lds_path(tn, oracle, slots, opt, hyper):
    """More than 32768 lookups in ragged slots (some empty, some with a handful of lookups,
    so that tiles of the partition kernels straddle many slots), non-zero labels, signs shared
    between slots, new signs in the second batch: remap and grouping through LDS (arrival-order
    grouping above 128 slots) against the oracle."""
    D = 8
    rng = np.random.default_rng(100 + slots)
    pair = Pair(tn, oracle, opt, D, hyper, reserve=400000, zero_init=True)
    vocab = 40000
    pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)).view(np.int64)
    pair.populate(pool[:30000].view(np.uint64))
    for step in range(2):
        values = []
        for s in range(slots):
            kind = s % 5
            n = 0 if kind == 0 else int(rng.integers(1, 8)) if kind == 1 else int(rng.integers(500, 4000))
            hot = pool[rng.integers(0, 50, n)]                 # a few signs everywhere
            cold = pool[rng.integers(0, vocab if step else 30000, n)]
            values.append(np.where(rng.random(n) < 0.3, hot, cold))
        assert sum(len(v) for v in values) > 40000
        counts = check_pull(pair, values)
        grads = synth.make_grads(counts, D, 0.01, seed=step)
        labels = [rng.integers(0, 3, len(v)).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        assert pair.assert_rows_match(all_signs(values)) > 0.99


def test_bound_ops_over_several_steps_without_waiting(tn, oracle):
    """Ops bound to their tensors once and called step after step: a pull runs behind
    the push before it without the host waiting in between, and a push whose signs were
    overwritten in place since the pull notices it."""
    D = 16
    rng = np.random.default_rng(33)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=400000)
    vocab = 30000
    base = pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    batches = [random_batch(rng, 6, 9000, vocab) for _ in range(3)]  # large enough for the remap through LDS
    bound = []
    for values in batches:
        gvalues = [dev(v) for v in values]
        gvars = [torch.zeros((len(v) + 1, D), device="cuda") for v in values]
        counts = [len(np.unique(v)) for v in values]
        grads = synth.make_grads(counts, D, 0.01, seed=len(bound))
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        pull = tn.ops.BoundSparseTablePull(gvars, gvalues, pair.h)
        push = tn.ops.BoundSparseTablePush(gvalues, [dev(g) for g in grads], [dev(l) for l in labels], pair.h)
        bound.append((values, gvalues, gvars, grads, labels, pull, push))
    for step in range(6):
        values, gvalues, gvars, grads, labels, pull, push = bound[step % 3]
        cvars = [np.zeros((len(v) + 1, D), np.float32) for v in values]
        rc, cmapped, counts = pair.o.pull_op(values, cvars)
        assert rc == 0
        gmapped = pull()
        for s in range(len(values)):
            assert (gmapped[s].cpu().numpy() == cmapped[s]).all()
            np.testing.assert_allclose(gvars[s].cpu().numpy(), cvars[s], rtol=RTOL, atol=ATOL)
        assert pair.o.push_op(values, grads, labels)[0] == 0
        push()
    tn.ops.sparse_table_sync(pair.h)
    pair.assert_rows_match(base)
    # same tensors, other signs in two places: the push must not use the pull's analysis
    values, gvalues, gvars, grads, labels, pull, push = bound[0]
    pull()
    pair.o.pull_op(values, [np.zeros((len(v) + 1, D), np.float32) for v in values])
    changed = [v.copy() for v in values]
    s0 = max(range(len(values)), key=lambda s: len(values[s]))
    other = int(np.flatnonzero(changed[s0] != changed[s0][0])[0])
    changed[s0][0], changed[s0][other] = changed[s0][other], changed[s0][0]  # same distinct signs, other order
    gvalues[s0].copy_(dev(changed[s0]))
    assert pair.o.push_op(changed, grads, labels)[0] == 0
    push()
    tn.ops.sparse_table_sync(pair.h)
    pair.assert_rows_match(base)


@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("change", ["one sign", "neighbours change places", "change places across tiles",
                                    "last lookup", "two signs to one"])
def test_a_push_notices_any_change_of_the_signs_since_the_pull(tn, oracle, change, exact):
    """After a pull through LDS the plan keeps fingerprints of the batch's signs, 16 bytes per 64 lookups, not the
    signs: a push whose value tensors were edited in place since the pull, in one place or with two signs
    changing places, must analyse its batch itself (the oracle is given the edited batch); the unedited batch is
    pushed on the pull's plan.  exact: with tn_sparse_table_set_exact_verify the pull keeps a copy of the signs
    as well and the push compares those."""
    from tensornet_amd import _lib

    D = 8
    rng = np.random.default_rng(55)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=200000)
    tn.core.set_sparse_table_exact_verify(pair.h, exact)
    verify = "k_verify_values<true, true>" if exact else "k_verify_values<true, false>"
    vocab = 20000
    base = pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    values = random_batch(rng, 3, 9000, vocab, ragged=False)  # 4.4 tiles of 2048 lookups a slot
    gvalues = [dev(v) for v in values]
    gvars = [torch.zeros((len(v) + 1, D), device="cuda") for v in values]
    labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
    glabels = [dev(l) for l in labels]

    def launched(fn):
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

    def step(edited, seed):
        tn.ops.sparse_table_pull(gvars, gvalues, pair.h)
        pair.o.pull_op(values, [np.zeros((len(v) + 1, D), np.float32) for v in values])
        for s, v in enumerate(edited):
            gvalues[s].copy_(dev(v))
        counts = [len(np.unique(v)) for v in edited]
        grads = synth.make_grads(counts, D, 0.01, seed=seed)
        assert pair.o.push_op(edited, grads, labels)[0] == 0
        names = launched(lambda: tn.ops.sparse_table_push(gvalues, [dev(g) for g in grads], glabels, pair.h))
        tn.ops.sparse_table_sync(pair.h)
        pair.assert_rows_match(base)
        for s, v in enumerate(values):
            gvalues[s].copy_(dev(v))
        return names

    names = step(values, 0)
    assert verify in names and "k_remap_insert" not in names  # fingerprints (or the copy), plan reused
    edited = [v.copy() for v in values]
    v = edited[1]
    if change == "one sign":
        v[4321] = next(int(x) for x in base.view(np.int64)[:2] if x != v[4321])  # another resident sign
    elif change == "neighbours change places":
        i = int(np.flatnonzero(v[:-1] != v[1:])[0])
        v[i], v[i + 1] = v[i + 1], v[i]
    elif change == "change places across tiles":
        j = int(np.flatnonzero(v[5000:] != v[10])[0]) + 5000
        v[10], v[j] = v[j], v[10]
    elif change == "last lookup":
        edited[2][-1] = edited[2][0] if edited[2][-1] != edited[2][0] else edited[2][1]
    else:
        a, b = int(v[100]), int(v[np.flatnonzero(v != v[100])[0]])
        v[v == b] = a
    assert any((e != o).any() for e, o in zip(edited, values))
    names = step(edited, 1)
    assert "k_remap_insert" in names  # the push worked the batch out itself
    assert verify in step(values, 2)


def test_detached_updates_are_seen_by_whatever_touches_the_table_next(tn, oracle):
    """tn_sparse_table_set_detached_updates: the update kernels of a large push (3 M lookups or more) run beside
    what the caller queues next.  Steps queued back to back without the host waiting in between -- the next pull's
    batch shares most signs with the push before it, so its variables must hold the updated rows; a small batch
    and a table-level call in between, a push of another batch than the pull's, and the final table -- against
    the oracle, which runs the same sequence one call after the other."""
    D = 16
    rng = np.random.default_rng(2024)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=10 ** 6)
    tn.core.set_sparse_table_detached_updates(pair.h, True)
    vocab = 300000
    base = pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    pool = base.view(np.int64)
    hot = pool[:40]

    def batch(slots, per):  # (every batch used below has 3 M lookups or more, but `small`)
        out = []
        for _ in range(slots):
            v = pool[(rng.random(per) ** 3 * vocab).astype(np.int64)]
            v[: len(hot)] = hot  # signs with a record in every slot: updated record after record, in slot order
            out.append(v)
        return out

    big = [batch(64, 50000) for _ in range(2)]  # 3.2 M lookups each: updates on the table's own streams
    assert all(sum(len(v) for v in b) >= 3 << 20 for b in big)
    small = batch(8, 1000)
    # (a batch with more slots and one with many more lookups than the push before it: their plans do not lie over
    # the plan the update kernels still read, so those pulls wait for the updates first)
    sequence = [big[0], big[1], small, big[0], batch(80, 42000), big[1], batch(64, 72000), big[0]]
    steps = []
    for k, values in enumerate(sequence):
        counts = [len(np.unique(v)) for v in values]
        steps.append(dict(values=values, gvalues=[dev(v) for v in values],
                          gvars=[torch.zeros((len(v) + 1, D), device="cuda") for v in values],
                          grads=synth.make_grads(counts, D, 0.01, seed=k),
                          labels=[(rng.random(len(v)) < 0.2).astype(np.int64) for v in values]))
    for st in steps:  # (the gradient tensors stay alive and untouched until the end: what the mode asks for)
        st["ggrads"] = [dev(g) for g in st["grads"]]
        st["glabels"] = [dev(l) for l in st["labels"]]
    # the device side, nothing waited for but what the pulls wait for themselves
    for k, st in enumerate(steps):
        st["gmapped"] = tn.ops.sparse_table_pull(st["gvars"], st["gvalues"], pair.h)
        tn.ops.sparse_table_push(st["gvalues"], st["ggrads"], st["glabels"], pair.h)
        if k == 1:  # a table-level call right behind a detached push: the rows it reads are the updated ones
            st["table_pull"] = tn.ops.table_pull(pair.h, dev(hot), D)
    # a push of another batch than the last pull's, behind a detached push
    other = batch(64, 50000)
    other_counts = [len(np.unique(v)) for v in other]
    other_grads = synth.make_grads(other_counts, D, 0.01, seed=99)
    other_labels = [np.zeros(len(v), np.int64) for v in other]
    gother = ([dev(v) for v in other], [dev(g) for g in other_grads], [dev(l) for l in other_labels])
    tn.ops.sparse_table_push(gother[0], gother[1], gother[2], pair.h)
    tn.ops.sparse_table_sync(pair.h)
    # the oracle, call by call
    for k, st in enumerate(steps):
        cvars = [np.zeros((len(v) + 1, D), np.float32) for v in st["values"]]
        rc, cmapped, counts = pair.o.pull_op(st["values"], cvars)
        assert rc == 0
        for s in range(len(cvars)):
            assert (st["gmapped"][s].cpu().numpy() == cmapped[s]).all()
            np.testing.assert_allclose(st["gvars"][s].cpu().numpy(), cvars[s], rtol=RTOL, atol=ATOL)
        assert pair.o.push_op(st["values"], st["grads"], st["labels"])[0] == 0
        if k == 1:
            cw, _, cf = pair.o.get_rows(hot.view(np.uint64))
            assert cf.all()
            np.testing.assert_allclose(st["table_pull"].cpu().numpy(), cw[:, :D], rtol=RTOL, atol=ATOL)
    assert pair.o.push_op(other, other_grads, other_labels)[0] == 0
    assert pair.assert_rows_match(base) > 0.99


@pytest.mark.parametrize("D", [8, 12, 64, 128])
@pytest.mark.parametrize("opt,hyper", [("AdaGrad", ADAGRAD_HP), ("Adam", ADAM_HP)])
def test_table_push_one_sign_with_very_many_records(tn, oracle, opt, hyper, D):
    """SparseTable::Push applies records in array order however often a sign repeats:
    a few records, a few hundred (one wavefront per sign) and more than fit in LDS; dims that
    divide the wavefront, one that does not, and one whose rows fill the staging 16 at a time."""
    rng = np.random.default_rng(13)
    pair = Pair(tn, oracle, opt, D, hyper)
    base = pair.populate(synth.splitmix64(np.arange(1, 41, dtype=np.uint64)))
    req = np.concatenate([np.full(5000, base[0]), np.full(300, base[1]), np.full(17, base[2]), np.full(15, base[3]),
                          base[rng.integers(4, 40, 700)]])
    req = req[rng.permutation(len(req))]
    n = len(req)
    infos = np.zeros(n, dtype=oracle.sign_info_dtype)
    infos["sign"] = req
    infos["batch_show"] = rng.integers(1, 4, n)
    infos["batch_click"] = rng.integers(0, 2, n)
    grads = (rng.standard_normal((n, D)) * 0.01).astype(np.float32)
    assert pair.o.push(infos, grads) == 0
    rec = tn.ops.make_sign_infos(dev(req.view(np.int64)), dev(infos["batch_show"].astype(np.int64)),
                                 dev(infos["batch_click"].astype(np.int64)))
    tn.ops.table_push(pair.h, rec, dev(grads))
    tn.ops.sparse_table_sync(pair.h)
    pair.assert_rows_match(base)


@pytest.mark.parametrize("slots", [70, 128, 129, 300])
def test_many_slots(tn, oracle, slots):
    """Slot counts on both sides of the 64- and 128-slot boundaries of the
    grouping by slot masks; a handful of signs occur in (nearly) every slot."""
    D = 16
    rng = np.random.default_rng(slots)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP)
    vocab = 400
    base = pair.populate(synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)))
    hot = base[:5].view(np.int64)
    for b in range(2):
        values = []
        for s_ in range(slots):
            n = int(rng.integers(0, 40))
            v = base.view(np.int64)[rng.integers(0, vocab, n)]
            values.append(np.concatenate([v, hot[: int(rng.integers(0, 6))]]))
        counts = check_pull(pair, values)
        grads = [(rng.standard_normal((int(u), D)) * 0.05).astype(np.float32) for u in counts]
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        pair.assert_rows_match(base)


def _hash32(signs):
    """Upper half of the 64-bit hash that places a sign among its slot's first-level buckets, among the
    second-level buckets and in the table (numpy restatement)."""
    x = np.asarray(signs, dtype=np.uint64).copy()
    with np.errstate(over="ignore"):
        x ^= x >> np.uint64(33)
        x *= np.uint64(0xFF51AFD7ED558CCD)
        x ^= x >> np.uint64(33)
        x *= np.uint64(0xC4CEB9FE1A85EC53)
        x ^= x >> np.uint64(33)
    return (x >> np.uint64(32)).astype(np.uint32)


def test_remap_falls_back_when_a_bucket_overflows(tn, oracle):
    """Large batches are remapped through hash tables in LDS: every tile of 2048 lookups hands its distinct signs
    to first-level buckets of fixed room (1536 records), chosen by a hash of the sign; a slot whose signs are
    crafted to fall into one bucket must still give the reference's ids and rows (the call is redone with more
    buckets and, as that cannot help here, on the global-table path)."""
    D = 8
    rng = np.random.default_rng(77)
    n_slot = 40000
    nb = (n_slot + 1149) // 1150  # buckets of the slot when no sign repeats inside a tile
    cand = rng.integers(0, 1 << 63, 400000, dtype=np.uint64)
    bucket = (_hash32(cand).astype(np.uint64) * np.uint64(nb)) >> np.uint64(32)
    crowd = cand[bucket == 0][:6000]
    assert len(crowd) == 6000
    filler = cand[bucket != 0][: n_slot - 6000]
    slot0 = rng.permutation(np.concatenate([crowd, filler])).view(np.int64)
    slot1 = rng.permutation(np.concatenate([crowd[:3000], filler[:5000]])).view(np.int64)
    values = [slot0, slot1]
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=200000)
    pair.populate(all_signs(values))
    counts = check_pull(pair, values)
    assert counts.tolist() == [len(np.unique(slot0)), len(np.unique(slot1))]
    grads = synth.make_grads(counts, D, 0.01)
    pair.push_op(values, grads, [np.ones(len(v), np.int64) for v in values])
    pair.assert_rows_match(all_signs(values))


def test_grouping_falls_back_when_a_second_level_bucket_overflows(tn, oracle):
    """The distinct records of all slots are grouped in buckets chosen by the sign's hash (room
    for 1536 records each); 2500 distinct signs crafted into one such bucket make the call fall
    back to the global-table path, with the reference's results."""
    D = 8
    rng = np.random.default_rng(78)
    slots, per_slot = 64, 1000
    nb2 = (slots * per_slot + 1023) // 1024
    cand = rng.integers(0, 1 << 63, 600000, dtype=np.uint64)
    bucket = (_hash32(cand).astype(np.uint64) * np.uint64(nb2)) >> np.uint64(32)
    crowd = cand[bucket == 0][:2560]
    assert len(crowd) == 2560
    filler = cand[bucket != 0]
    values = []
    for s in range(slots):
        mine = np.concatenate([crowd[s * 40:(s + 1) * 40], filler[s * 900:s * 900 + 960]])
        values.append(rng.permutation(mine).view(np.int64))
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=300000)
    pair.populate(all_signs(values))
    counts = check_pull(pair, values)
    grads = synth.make_grads(counts, D, 0.01)
    pair.push_op(values, grads, [np.ones(len(v), np.int64) for v in values])
    pair.assert_rows_match(all_signs(values))


def test_cfg3_full_batch_against_the_oracle(tn, oracle):
    """One whole cfg3 batch (16384 x 100 slots, ~5 M lookups, ~2 M distinct per slot, ~1.1 M
    distinct signs) through pull and push on both sides: every mapped id and pulled row bit for
    bit, every updated row within the tolerance (and nearly all of them bit for bit).  The
    resident set is the batch's own signs (the oracle cannot hold 5e8 rows)."""
    cfg = synth.CONFIGS["cfg3"]
    D = cfg["dim"]
    values = synth.make_batch(cfg, 2)
    signs = all_signs(values)
    pair = Pair(tn, oracle, "AdaGrad", D, cfg["hyper"], reserve=3 * 10 ** 6)
    pair.populate(signs)
    counts = check_pull(pair, values)
    assert sum(len(v) for v in values) > 4.9e6 and int(counts.sum()) > 1.9e6
    grads = synth.make_grads(counts, D, cfg["grad_sigma"], seed=9)
    rng = np.random.default_rng(9)
    labels = [(rng.random(len(v)) < 0.05).astype(np.int64) for v in values]
    pair.push_op(values, grads, labels)
    assert pair.assert_rows_match(signs) > 0.99
    check_pull(pair, values)


def test_two_pushes_on_one_pull_count_their_own_clicks(tn, oracle):
    """A pull followed by two pushes of the same batch with different labels (the plan of the
    pull serves both): every push adds its own click sums, not the sum of both."""
    D = 8
    rng = np.random.default_rng(77)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, use_cvm=True, reserve=200000)
    vocab = 20000
    pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)).view(np.int64)
    pair.populate(pool.view(np.uint64))
    values = [pool[rng.integers(0, vocab, 3000)] for _ in range(16)]  # 48000 lookups: the LDS path
    counts = check_pull(pair, values, loose_col=D + 1)
    for push in range(2):
        grads = [(rng.standard_normal((int(u), D + 2)) * 0.01).astype(np.float32) for u in counts]
        labels = [rng.integers(0, 3, len(v)).astype(np.int64) for v in values]
        pair.push_op(values, grads, labels)
        pair.assert_rows_match(all_signs(values))


def test_two_tables_driven_from_two_host_threads(tn, oracle):
    """Different tables may be hit concurrently (TF runs ComputeAsync from inter-op threads,
    core/kernels/sparse_table_ops.cc:203-236): two host threads, each with its own stream and
    table, run pull + push steps at the same time; afterwards the oracle replays both
    sequences and must see the same mapped ids, pulled rows and final tables."""
    import threading

    specs = [("AdaGrad", 8, ADAGRAD_HP, 21), ("Adam", 16, ADAM_HP, 22)]
    vocab, steps = 30000, 4
    pool = synth.splitmix64(np.arange(1, vocab + 1, dtype=np.uint64)).view(np.int64)
    pairs, plans = [], []
    for opt, D, hp, seed in specs:
        pair = Pair(tn, oracle, opt, D, hp, reserve=300000, zero_init=True)
        pair.populate(pool[:20000].view(np.uint64))
        rng = np.random.default_rng(seed)
        batches = []
        for _ in range(steps):
            values = [pool[rng.integers(0, vocab, int(rng.integers(2000, 4000)))] for _ in range(16)]  # LDS path
            labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
            batches.append((values, labels, int(rng.integers(1 << 30))))
        pairs.append(pair)
        plans.append(batches)
    results = [[] for _ in pairs]
    errors = []

    def drive(k):
        try:
            pair = pairs[k]
            with torch.cuda.stream(torch.cuda.Stream()):
                for values, labels, gseed in plans[k]:
                    gvars = [torch.full((len(v) + 1, pair.wf), -7.0, device="cuda") for v in values]
                    mapped = tn.ops.sparse_table_pull(gvars, [dev(v) for v in values], pair.h)
                    counts = tn.ops.sparse_table_last_unique_counts(pair.h, len(values))
                    grads = synth.make_grads(np.array(counts), pair.wf, 0.01, seed=gseed)
                    tn.ops.sparse_table_push([dev(v) for v in values], [dev(g) for g in grads],
                                             [dev(l) for l in labels], pair.h)
                    tn.ops.sparse_table_sync(pair.h)
                    # statistics of BOTH tables while the other thread drives its own: a key count waits
                    # for its table's work only (a device-wide wait here would serialise the two threads)
                    for other in pairs:
                        assert 20000 <= tn.core.sparse_table_key_count(other.h) <= vocab
                    results[k].append(([m.cpu().numpy() for m in mapped], [v.cpu().numpy() for v in gvars], counts,
                                       grads))
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=drive, args=(k,)) for k in range(len(pairs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for k, pair in enumerate(pairs):
        for (values, labels, _), (gm, gv, counts, grads) in zip(plans[k], results[k]):
            cvars = [np.full((len(v) + 1, pair.wf), -7.0, np.float32) for v in values]
            rc, cm, ccounts = pair.o.pull_op(values, cvars)
            assert rc == 0 and ccounts.tolist() == counts
            for s in range(len(values)):
                assert (gm[s] == cm[s]).all()
                assert (gv[s].view(np.int32) == cvars[s].view(np.int32)).all()
            rc, _ = pair.o.push_op(values, grads, labels)
            assert rc == 0
        assert pair.assert_rows_match(all_signs([v for b in plans[k] for v in b[0]])) > 0.99


def _mix64(x):
    m = (1 << 64) - 1
    x ^= x >> 33
    x = (x * 0xff51afd7ed558ccd) & m
    x ^= x >> 33
    x = (x * 0xc4ceb9fe1a85ec53) & m
    x ^= x >> 33
    return x


def test_probe_chains_wrap_around_the_end_of_the_table(tn, oracle):
    """Collisions: signs whose home slots all lie in the last group of 8 slots of the table, three
    times as many as the group holds, so that their probe sequences run over the end of the
    table into its first groups; pulled, pushed, pulled again and found again by a push of
    another batch (probe without insert)."""
    D = 8
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=100, zero_init=True)
    pair.populate(synth.splitmix64(np.arange(1, 4, dtype=np.uint64)))  # allocates the table
    cap = tn.core.sparse_table_capacity(pair.h)
    assert cap % 8 == 0 and cap < 400
    rng = np.random.default_rng(3)
    crowd = []
    while len(crowd) < 24:
        s = int(rng.integers(1, 1 << 62))
        if (_mix64(s) * cap) >> 64 >= cap - 8:
            crowd.append(s)
    signs = np.array(crowd, dtype=np.int64)
    values = [signs[:16], signs[8:]]  # overlapping slots: 8 of the signs get two records
    counts = check_pull(pair, values)
    assert tn.core.sparse_table_capacity(pair.h) == cap  # no growth: the chains are what is tested
    grads = synth.make_grads(counts, D, 0.01, seed=5)
    pair.push_op(values, grads, [np.ones(len(v), np.int64) for v in values])
    assert pair.assert_rows_match(all_signs(values)) > 0.99
    check_pull(pair, values)
    other = [signs[::-1].copy()]  # another batch than the last pull's: its plan is built by the push
    counts = pair.o.pull_op(other, [np.zeros((len(signs) + 1, pair.wf), np.float32)])[2]
    grads = synth.make_grads(counts, D, 0.01, seed=6)
    pair.push_op(other, grads, [np.zeros(len(signs), np.int64)])
    assert pair.assert_rows_match(all_signs(values)) > 0.99


def test_batch_with_more_distinct_signs_than_the_recent_ones(tn, oracle):
    """The second-level buckets of the grouping are sized from the share of distinct records the
    recent pulls had.  Twenty batches of heavily repeated signs, then one of the same size in which
    every lookup is distinct: it overflows buckets, takes the fallback path, and everything
    still equals the oracle; the batch after it runs on buckets sized for the worst case again."""
    D = 8
    rng = np.random.default_rng(41)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=400000, zero_init=True)
    pool = synth.splitmix64(np.arange(1, 200001, dtype=np.uint64)).view(np.int64)
    pair.populate(pool[:1000].view(np.uint64))
    slots, per = 16, 4000
    for step in range(20):
        values = [pool[rng.integers(0, 300, per)] for _ in range(slots)]  # 64000 lookups, a few hundred signs
        if step % 7 == 0:
            check_pull(pair, values)
        else:
            tn.ops.sparse_table_pull([torch.empty((per + 1, D), device="cuda") for _ in values],
                                     [dev(v) for v in values], pair.h)
    for step in range(2):
        values = [pool[1000 + (step * slots + s) * per:1000 + (step * slots + s + 1) * per] for s in range(slots)]
        counts = check_pull(pair, values)  # every lookup a new sign
        assert counts.tolist() == [per] * slots
        grads = synth.make_grads(counts, D, 0.01, seed=step)
        pair.push_op(values, grads, [np.zeros(per, np.int64) for _ in values])
        assert pair.assert_rows_match(all_signs(values)) > 0.99


@pytest.mark.gpu
def test_batch_beyond_the_sizes_the_fused_scans_cover(tn, oracle):
    """18 M lookups in one call: more tiles and more second-level buckets than the ranking
    and member-list kernels add up themselves, so the separate scan kernels run.  Too large
    for the CPU oracle in seconds: the same size-independent properties as for cfg3."""
    D, N, per_slot = 16, 24, 750000
    opt = tn.core.AdaGrad(learning_rate=0.01, initial_g2sum=0.1)
    h = tn.core.create_sparse_table(opt, "", D, False, "")
    tn.core.reserve_sparse_table(h, 4 * 10 ** 6)
    gen = torch.Generator(device="cuda").manual_seed(5)
    # a shared vocabulary, so that signs repeat inside a slot and across slots
    gvalues = [synth.splitmix64_torch(torch.randint(1, 3 * 10 ** 6, (per_slot + 1000 * s,), generator=gen,
                                                    device="cuda")) for s in range(N)]
    L = sum(len(v) for v in gvalues)
    assert L > 8192 * 2048
    uniq = torch.unique(torch.cat(gvalues))
    w0 = synth.snapshot_rows_torch(uniq, D)
    tn.ops.table_load_rows(h, uniq, w0)
    rows = [len(v) + 1 for v in gvalues]
    gvars = [torch.full((r, D), 9.0, device="cuda") for r in rows]
    mapped = tn.ops.sparse_table_pull(gvars, gvalues, h)
    counts = tn.ops.sparse_table_last_unique_counts(h, N)
    for s in (0, 7, N - 1):
        v, m = gvalues[s], mapped[s]
        u, inv = torch.unique(v, return_inverse=True)
        assert counts[s] == u.numel() == int(m.max()) + 1
        first = torch.full((u.numel(),), len(v), dtype=torch.int64, device="cuda")
        first.scatter_reduce_(0, inv, torch.arange(len(v), device="cuda"), reduce="amin")
        first_by_id = torch.empty_like(first)
        first_by_id[m[first]] = first
        assert bool((first_by_id[1:] > first_by_id[:-1]).all())
        assert torch.equal(m, m[first][inv])
        assert torch.equal(gvars[s][m], synth.snapshot_rows_torch(v, D))
        assert bool((gvars[s][counts[s]:] == 9.0).all())
    # a constant gradient: a sign present in k slots gets k sequential Applies
    g = 0.5
    grads = [torch.full((c, D), g, device="cuda") for c in counts]
    labels = [torch.ones_like(v) for v in gvalues]
    tn.ops.sparse_table_push(gvalues, grads, labels, h)
    tn.ops.sparse_table_sync(h)
    w2, st2, found = tn.ops.table_export_rows(h, uniq)
    assert bool(found.all())
    k = torch.zeros(uniq.numel(), device="cuda")
    for v in gvalues:
        k[torch.searchsorted(uniq, torch.unique(v))] += 1
    np.testing.assert_allclose(st2[:, 0].cpu().numpy(), (0.1 + k * g * g).cpu().numpy(), rtol=1e-5)
    assert float(st2[:, 1].double().sum()) == float(L) == float(st2[:, 2].double().sum())  # shows, clicks
    steps = torch.arange(1, int(k.max()) + 1, device="cuda", dtype=torch.float64)
    cum = torch.cumsum(0.01 * g / torch.sqrt(0.1 + steps * g * g), 0)
    expect = w0.double() - cum[(k - 1).long()][:, None]
    np.testing.assert_allclose(w2.cpu().numpy(), expect.cpu().numpy(), rtol=RTOL, atol=1e-6)


@pytest.mark.gpu
def test_calls_on_another_stream_wait_for_the_last_pull(tn, oracle):
    """A large pull returns when its counts and errors are on the host, while the copy of the
    pulled rows may still be running on its stream.  A push and a second pull issued at once on
    ANOTHER stream (which reuse the table's scratch memory) must wait for it by themselves."""
    D = 16
    rng = np.random.default_rng(77)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=1200000, zero_init=True)
    pool = synth.splitmix64(np.arange(1, 600001, dtype=np.uint64)).view(np.int64)
    pair.populate(pool.view(np.uint64))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for step in range(3):
        # step 0: a batch large enough for the side streams (more than 3 M lookups), step 1: a small one, step 2:
        # one for the path of few launches (every slot within 4096 lookups), whose pull also returns before its
        # last kernels have run
        per_slot = ((200000, 230000), (3000, 6000), (500, 3000))[step]
        values = [pool[rng.integers(0, 600000, int(rng.integers(*per_slot)))] for _ in range(16)]
        assert (sum(len(v) for v in values) > 3 << 20) == (step == 0)
        rows = [len(v) + 1 for v in values]
        cvars = [np.full((r, pair.wf), -7.0, np.float32) for r in rows]
        rc, cmapped, counts = pair.o.pull_op(values, cvars)
        assert rc == 0
        grads = synth.make_grads(counts, D, 0.01, seed=step)
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        assert pair.o.push_op(values, grads, labels)[0] == 0
        cvars2 = [np.full((r, pair.wf), -7.0, np.float32) for r in rows]
        assert pair.o.pull_op(values, cvars2)[0] == 0
        gvalues, ggrads, glabels = [dev(v) for v in values], [dev(g) for g in grads], [dev(l) for l in labels]
        gvars = [torch.full((r, pair.wf), -7.0, device="cuda") for r in rows]
        gvars2 = [torch.full((r, pair.wf), -7.0, device="cuda") for r in rows]
        torch.cuda.synchronize()
        with torch.cuda.stream(s1):
            gmapped = tn.ops.sparse_table_pull(gvars, gvalues, pair.h)
        with torch.cuda.stream(s2):  # no synchronisation in between
            tn.ops.sparse_table_push(gvalues, ggrads, glabels, pair.h)
            gmapped2 = tn.ops.sparse_table_pull(gvars2, gvalues, pair.h)
        torch.cuda.synchronize()
        for s in range(len(values)):
            assert np.array_equal(gmapped[s].cpu().numpy(), cmapped[s])
            assert np.array_equal(gmapped2[s].cpu().numpy(), cmapped[s])
            np.testing.assert_allclose(gvars[s].cpu().numpy(), cvars[s], rtol=RTOL, atol=ATOL)
            np.testing.assert_allclose(gvars2[s].cpu().numpy(), cvars2[s], rtol=RTOL, atol=ATOL)


@pytest.mark.gpu
def test_pull_on_another_stream_waits_for_the_updates_of_a_small_push(tn, oracle):
    """The push of a small batch returns when its signs are compared, with its update kernel still running on
    its stream.  A pull issued at once on ANOTHER stream reads the rows that kernel writes: it has to order
    itself behind it (table-level and op-level pulls alike)."""
    D = 16
    rng = np.random.default_rng(79)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=400000, zero_init=True)
    pool = synth.splitmix64(np.arange(1, 100001, dtype=np.uint64)).view(np.int64)
    pair.populate(pool.view(np.uint64))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for step in range(4):
        values = [pool[rng.integers(0, 100000, int(rng.integers(2000, 4000)))] for _ in range(24)]
        rows = [len(v) + 1 for v in values]
        cvars = [np.full((r, pair.wf), -7.0, np.float32) for r in rows]
        rc, cmapped, counts = pair.o.pull_op(values, cvars)
        assert rc == 0
        grads = synth.make_grads(counts, D, 0.05, seed=step)
        labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
        assert pair.o.push_op(values, grads, labels)[0] == 0
        cvars2 = [np.full((r, pair.wf), -7.0, np.float32) for r in rows]
        assert pair.o.pull_op(values, cvars2)[0] == 0
        gvalues, ggrads, glabels = [dev(v) for v in values], [dev(g) for g in grads], [dev(l) for l in labels]
        gvars = [torch.full((r, pair.wf), -7.0, device="cuda") for r in rows]
        gvars2 = [torch.full((r, pair.wf), -7.0, device="cuda") for r in rows]
        some = np.unique(np.concatenate(values))[:5000]
        gsome = dev(some)
        torch.cuda.synchronize()
        with torch.cuda.stream(s2):
            tn.ops.sparse_table_pull(gvars, gvalues, pair.h)
            tn.ops.sparse_table_push(gvalues, ggrads, glabels, pair.h)
        with torch.cuda.stream(s1):  # no synchronisation in between
            if step % 2 == 0:
                gmapped2 = tn.ops.sparse_table_pull(gvars2, gvalues, pair.h)
            else:
                table_rows = tn.ops.table_pull(pair.h, gsome, D)
        torch.cuda.synchronize()
        if step % 2 == 0:
            for s in range(len(values)):
                assert np.array_equal(gmapped2[s].cpu().numpy(), cmapped[s])
                np.testing.assert_allclose(gvars2[s].cpu().numpy(), cvars2[s], rtol=RTOL, atol=ATOL)
        else:
            cw, _, cf = pair.o.get_rows(some.view(np.uint64))
            assert cf.all()
            np.testing.assert_allclose(table_rows.cpu().numpy(), cw[:, :D], rtol=RTOL, atol=ATOL)


@pytest.mark.gpu
def test_push_on_another_stream_waits_for_an_asynchronous_pull(tn, oracle):
    """With asynchronous pulls the op only enqueues its kernels.  A push of the same batch issued at once on
    ANOTHER stream reads the plan those kernels are still building: it has to wait for the pull's stream by
    itself (as a second pull does)."""
    D = 16
    rng = np.random.default_rng(78)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=400000, zero_init=True)
    pool = synth.splitmix64(np.arange(1, 200001, dtype=np.uint64)).view(np.int64)
    pair.populate(pool[:150000].view(np.uint64))
    tn.core.set_sparse_table_async(pair.h, True)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    try:
        for step in range(3):
            values = [pool[rng.integers(0, 200000, int(rng.integers(20000, 40000)))] for _ in range(12)]
            rows = [len(v) + 1 for v in values]
            cvars = [np.full((r, pair.wf), -7.0, np.float32) for r in rows]
            rc, cmapped, counts = pair.o.pull_op(values, cvars)
            assert rc == 0
            grads = synth.make_grads(counts, D, 0.01, seed=step)
            labels = [rng.integers(0, 2, len(v)).astype(np.int64) for v in values]
            assert pair.o.push_op(values, grads, labels)[0] == 0
            gvalues, ggrads, glabels = [dev(v) for v in values], [dev(g) for g in grads], [dev(l) for l in labels]
            gvars = [torch.full((r, pair.wf), -7.0, device="cuda") for r in rows]
            torch.cuda.synchronize()
            with torch.cuda.stream(s1):
                gmapped = tn.ops.sparse_table_pull(gvars, gvalues, pair.h)
            with torch.cuda.stream(s2):  # no synchronisation in between
                tn.ops.sparse_table_push(gvalues, ggrads, glabels, pair.h)
            tn.ops.sparse_table_sync(pair.h)
            torch.cuda.synchronize()
            assert tn.ops.sparse_table_last_unique_counts(pair.h, len(values)) == counts.tolist()
            for s in range(len(values)):
                assert np.array_equal(gmapped[s].cpu().numpy(), cmapped[s])
                np.testing.assert_allclose(gvars[s].cpu().numpy(), cvars[s], rtol=RTOL, atol=ATOL)
            assert pair.assert_rows_match(all_signs(values)) > 0.99
    finally:
        tn.core.set_sparse_table_async(pair.h, False)


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [0, 1, 3, 4, 5, 7, 2047])
def test_batch_sizes_around_the_tile_and_vector_boundaries(tn, oracle, extra):
    """The ranking kernels take 4 or 8 lookups per thread with 16-byte accesses and handle the last,
    incomplete group one by one: total sizes of every remainder, slot boundaries that are no
    multiple of the vector widths."""
    D = 8
    rng = np.random.default_rng(900 + extra)
    pair = Pair(tn, oracle, "AdaGrad", D, ADAGRAD_HP, reserve=200000, zero_init=True)
    pool = synth.splitmix64(np.arange(1, 20001, dtype=np.uint64)).view(np.int64)
    pair.populate(pool[:15000].view(np.uint64))
    total = 16 * 2048 + extra
    cuts = np.sort(rng.choice(np.arange(1, total), 6, replace=False))
    lens = np.diff(np.concatenate([[0], cuts, [total]]))
    lens = np.concatenate([lens[:3], [0], lens[3:]])  # an empty slot in the middle
    values = [pool[rng.integers(0, 20000, int(n))] for n in lens]
    assert sum(len(v) for v in values) == total
    counts = check_pull(pair, values)
    grads = synth.make_grads(counts, D, 0.01, seed=extra)
    labels = [rng.integers(-1, 3, len(v)).astype(np.int64) for v in values]
    pair.push_op(values, grads, labels)
    assert pair.assert_rows_match(all_signs(values)) > 0.99


@pytest.mark.gpu
def test_variable_too_small_is_reported_on_a_large_batch(tn, oracle):
    """More than 3 M lookups (the pull returns while its last kernel still runs): a variable with
    fewer rows than its slot has distinct signs is still TN_ERR_VAR_CAPACITY (sparse_table_ops.cc:136),
    nothing is written beyond its rows, and the table serves the next call."""
    D = 16
    opt = tn.core.AdaGrad(learning_rate=0.01, initial_g2sum=0.1)
    h = tn.core.create_sparse_table(opt, "", D, False, "")
    tn.core.reserve_sparse_table(h, 10 ** 6)
    gen = torch.Generator(device="cuda").manual_seed(9)
    gvalues = [synth.splitmix64_torch(torch.randint(1, 500000, (210000,), generator=gen, device="cuda"))
               for _ in range(16)]
    assert sum(len(v) for v in gvalues) > 3 << 20
    rows = [len(v) + 1 for v in gvalues]
    small = 1000
    guard = torch.full((small + 64, D), 9.0, device="cuda")  # the variable is its first `small` rows
    gvars = [torch.full((r, D), 9.0, device="cuda") for r in rows]
    gvars[3] = guard[:small]
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.sparse_table_pull(gvars, gvalues, h)
    assert e.value.code == 4
    torch.cuda.synchronize()
    assert bool((guard[small:] == 9.0).all())
    gvars[3] = torch.full((rows[3], D), 9.0, device="cuda")
    mapped = tn.ops.sparse_table_pull(gvars, gvalues, h)
    counts = tn.ops.sparse_table_last_unique_counts(h, 16)
    torch.cuda.synchronize()
    for s in (0, 3, 15):
        assert counts[s] == torch.unique(gvalues[s]).numel() == int(mapped[s].max()) + 1
