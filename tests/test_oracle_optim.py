"""Pins the oracle's sparse optimizer rows (A3, A4, A6, A7a-c) without the
reference: hand-computed exact known answers, numpy evaluations of the
reference formulas with explicit float32 / float64 casts, float64 closed
forms, and special cases that reduce to textbook rules."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
f32 = np.float32
SIGN = np.asarray([0x1234567890ABCDEF], dtype=np.uint64)


def kat():
    with open(os.path.join(HERE, "golden", "optim_kat.json")) as f:
        return json.load(f)


def one_info(oracle, show, click=0, sign=SIGN[0]):
    info = np.zeros(1, dtype=oracle.sign_info_dtype)
    info["sign"] = sign
    info["batch_show"] = show
    info["batch_click"] = click
    return info


def i2f(i):
    return np.asarray([i], dtype=np.int32).view(np.float32)[0]


def f2i(f):
    return int(np.asarray([f], dtype=np.float32).view(np.int32)[0])


# ------------------------------------------------------------ known answers
def test_adagrad_known_answers(oracle):
    for c in kat()["adagrad"]:
        t = oracle.Table(oracle.ADAGRAD, c["dim"], buckets=64, **c["hyper"])
        st0 = np.asarray(c["state0"][:3] + [i2f(c["state0"][3])], dtype=np.float32)
        t.set_rows(SIGN, np.asarray([c["w0"]], dtype=np.float32), st0[None, :])
        assert t.push(one_info(oracle, c["show"], c["click"]), np.asarray([c["grad"]], dtype=np.float32)) == 0
        w, st, found = t.get_rows(SIGN)
        assert found[0] == 1
        assert w[0].tolist() == c["w1"]
        assert st[0, :3].tolist() == c["state1"][:3]
        assert f2i(st[0, 3]) == c["state1"][3]


def test_adam_known_answers(oracle):
    for c in kat()["adam"]:
        D = c["dim"]
        t = oracle.Table(oracle.ADAM, D, buckets=64, **c["hyper"])
        st0 = np.asarray(c["m0"] + c["v0"] + [0.0, i2f(0)], dtype=np.float32)
        t.set_rows(SIGN, np.asarray([c["w0"]], dtype=np.float32), st0[None, :])
        t.push(one_info(oracle, c["show"]), np.asarray([c["grad"]], dtype=np.float32))
        w, st, _ = t.get_rows(SIGN)
        assert w[0].tolist() == c["w1"]
        assert st[0, :D].tolist() == c["m1"]
        assert st[0, D:2 * D].tolist() == c["v1"]
        assert f2i(st[0, 2 * D + 1]) == c["delta_show1"]


def test_ftrl_known_answers(oracle):
    for c in kat()["ftrl"]:
        D = c["dim"]
        t = oracle.Table(oracle.FTRL, D, buckets=64, **c["hyper"])
        st0 = np.asarray(c["z0"] + c["n0"] + [0.0, i2f(0)], dtype=np.float32)
        t.set_rows(SIGN, np.asarray([c["w0"]], dtype=np.float32), st0[None, :])
        t.push(one_info(oracle, c["show"]), np.asarray([c["grad"]], dtype=np.float32))
        w, st, _ = t.get_rows(SIGN)
        assert w[0].tolist() == c["w1"], c["_why"]
        assert st[0, :D].tolist() == c["z1"]
        assert st[0, D:2 * D].tolist() == c["n1"]
        assert f2i(st[0, 2 * D + 1]) == c["delta_show1"]


# ------------------------------------------- numpy evaluation, explicit casts
def np_adagrad(w, st, g, show, click, lr, eps, use_cvm=False):
    """ada_grad_kernel.cc:105-129 with every promotion spelled out."""
    D = len(g)
    w = w.copy()
    g2sum, sh, ck = f32(st[0]), f32(st[1]), f32(st[2])
    sh = f32(sh + f32(show))
    ck = f32(ck + f32(click))
    add = np.float64(0)
    for i in range(D):
        add = add + np.float64(f32(g[i] * g[i]))
    g2sum = f32(np.float64(g2sum) + add / np.float64(D))
    den = f32(f32(eps) + np.sqrt(g2sum, dtype=np.float32))
    for i in range(D):
        w[i] = f32(w[i] - f32(f32(f32(lr) * g[i]) / den))
    if use_cvm:
        w[D] = sh
        w[D + 1] = f32(np.log(f32(ck + f32(1)), dtype=np.float32) - np.log(f32(sh + f32(1)), dtype=np.float32))
    return w, np.asarray([g2sum, sh, ck, i2f(0)], dtype=np.float32)


def np_adam(w, m, v, g, lr, b1, b2, eps):
    """adam_kernel.cc:112-125: no bias correction, (1 - beta) evaluated in float."""
    lr, b1, b2, eps = f32(lr), f32(b1), f32(b2), f32(eps)
    c1, c2 = f32(f32(1) - b1), f32(f32(1) - b2)
    m = (b1 * m + c1 * g).astype(np.float32)
    v = (b2 * v + (c2 * g).astype(np.float32) * g).astype(np.float32)
    w = (w - (lr * m).astype(np.float32) / (eps + np.sqrt(v, dtype=np.float32))).astype(np.float32)
    return w, m, v


def np_ftrl(w, z, n, g, lr, beta, l1, l2):
    """ftrl_kernel.cc:57-80."""
    lr, beta, l1, l2 = f32(lr), f32(beta), f32(l1), f32(l2)
    w, z, n = w.copy(), z.copy(), n.copy()
    for i in range(len(g)):
        g2 = f32(g[i] * g[i])
        z[i] = f32(z[i] + f32(g[i] - f32(f32(lr * f32(np.sqrt(f32(n[i] + g2)) - np.sqrt(n[i]))) * w[i])))
        n[i] = f32(n[i] + g2)
        if abs(z[i]) <= l1:
            w[i] = f32(0)
        else:
            w[i] = f32(f32(-1) / f32(f32(f32(beta + np.sqrt(n[i])) * lr) + l2))
            if z[i] > 0:
                w[i] = f32(w[i] * f32(z[i] - l1))
            else:
                w[i] = f32(w[i] * f32(z[i] + l1))
    return w, z, n


@pytest.mark.parametrize("dim", [1, 8, 16, 64])
@pytest.mark.parametrize("use_cvm", [False, True])
def test_adagrad_matches_cast_exact_numpy(oracle, dim, use_cvm):
    rng = np.random.default_rng(dim)
    lr, eps = 0.01, 1e-8
    t = oracle.Table(oracle.ADAGRAD, dim, use_cvm=use_cvm, buckets=64, learning_rate=lr, initial_g2sum=0.1, epsilon=eps)
    w = rng.uniform(-0.01, 0.01, t.wf).astype(np.float32)
    st = np.asarray([0.1, 0, 0, i2f(3)], dtype=np.float32)
    t.set_rows(SIGN, w[None, :], st[None, :])
    for step in range(5):  # repeated Applies to one key
        g = (rng.standard_normal(t.wf) * 0.01).astype(np.float32)
        show, click = int(rng.integers(1, 9)), int(rng.integers(0, 3))
        t.push(one_info(oracle, show, click), g[None, :])
        w, st = np_adagrad(w, st, g[:dim], show, click, lr, eps, use_cvm)
        ow, ost, _ = t.get_rows(SIGN)
        assert (ow[0, :dim] == w[:dim]).all(), (step, ow[0] - w)
        if use_cvm:  # libm's logf and numpy's float32 log may differ in the last bit
            assert ow[0, dim] == w[dim]
            np.testing.assert_allclose(ow[0, dim + 1], w[dim + 1], rtol=1e-6)
        assert (ost[0].view(np.int32) == st.view(np.int32)).all()


@pytest.mark.parametrize("dim", [1, 16, 64])
def test_adam_matches_cast_exact_numpy(oracle, dim):
    rng = np.random.default_rng(100 + dim)
    hp = dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8)
    t = oracle.Table(oracle.ADAM, dim, buckets=64, **hp)
    w = rng.uniform(-0.01, 0.01, dim).astype(np.float32)
    m = np.zeros(dim, dtype=np.float32)
    v = np.zeros(dim, dtype=np.float32)
    t.set_rows(SIGN, w[None, :])
    shows = 0
    for step in range(5):
        g = (rng.standard_normal(dim) * 1e-3).astype(np.float32)
        t.push(one_info(oracle, step + 1), g[None, :])
        shows += step + 1
        w, m, v = np_adam(w, m, v, g, hp["learning_rate"], hp["beta1"], hp["beta2"], hp["epsilon"])
        ow, ost, _ = t.get_rows(SIGN)
        assert (ow[0] == w).all()
        assert (ost[0, :dim] == m).all() and (ost[0, dim:2 * dim] == v).all()
        assert f2i(ost[0, 2 * dim + 1]) == shows


@pytest.mark.parametrize("dim", [1, 8])
def test_ftrl_matches_cast_exact_numpy(oracle, dim):
    rng = np.random.default_rng(200 + dim)
    hp = dict(learning_rate=0.05, beta=1.0, lambda1=1.0, lambda2=1.0)
    t = oracle.Table(oracle.FTRL, dim, buckets=64, **hp)
    w = rng.uniform(-0.01, 0.01, dim).astype(np.float32)
    z = np.zeros(dim, dtype=np.float32)
    n = np.zeros(dim, dtype=np.float32)
    t.set_rows(SIGN, w[None, :])
    inside = outside = 0
    for step in range(40):
        g = (rng.standard_normal(dim) * 0.6).astype(np.float32)
        t.push(one_info(oracle, 1), g[None, :])
        w, z, n = np_ftrl(w, z, n, g, hp["learning_rate"], hp["beta"], hp["lambda1"], hp["lambda2"])
        inside += int((np.abs(z) <= 1.0).sum())
        outside += int((np.abs(z) > 1.0).sum())
        ow, ost, _ = t.get_rows(SIGN)
        assert (ow[0] == w).all()
        assert (ost[0, :dim] == z).all() and (ost[0, dim:2 * dim] == n).all()
    assert inside > 0 and outside > 0  # both branches of the threshold were taken


# ------------------------------------------------- float64 closed forms etc.
def test_adagrad_float64_closed_form(oracle):
    """g2sum after k Applies = g2sum0 + sum_k mean(g_k^2); each step moves w by
    -lr*g/sqrt(g2sum) (eps negligible).  A dropped 1/D, a per-element g2sum or a
    wrong sign would all fail."""
    D, lr = 16, 0.01
    rng = np.random.default_rng(7)
    t = oracle.Table(oracle.ADAGRAD, D, buckets=64, learning_rate=lr, initial_g2sum=0.1, epsilon=1e-8)
    w0 = rng.uniform(-0.01, 0.01, D).astype(np.float32)
    t.set_rows(SIGN, w0[None, :])
    w = w0.astype(np.float64)
    g2 = 0.1
    for _ in range(10):
        g = (rng.standard_normal(D) * 0.05).astype(np.float32)
        t.push(one_info(oracle, 1), g[None, :])
        g2 += float(np.mean(g.astype(np.float64) ** 2))
        w = w - lr * g.astype(np.float64) / (1e-8 + np.sqrt(g2))
    ow, ost, _ = t.get_rows(SIGN)
    np.testing.assert_allclose(ow[0], w, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(ost[0, 0], g2, rtol=1e-6)
    assert ost[0, 1] == 10.0


def test_adam_beta_zero_is_sign_descent(oracle):
    """beta1 = beta2 = eps = 0: m = g, v = g^2, w -= lr * g/|g| (textbook reduction)."""
    D, lr = 8, 0.125
    t = oracle.Table(oracle.ADAM, D, buckets=64, learning_rate=lr, beta1=0.0, beta2=0.0, epsilon=0.0)
    w0 = np.linspace(-1, 1, D).astype(np.float32)
    t.set_rows(SIGN, w0[None, :])
    g = np.asarray([3, -2, 0.5, -0.25, 7, -9, 1, -1], dtype=np.float32)
    t.push(one_info(oracle, 1), g[None, :])
    ow, _, _ = t.get_rows(SIGN)
    np.testing.assert_array_equal(ow[0], w0 - lr * np.sign(g))


def test_ftrl_with_unit_rate_is_textbook_ftrl_proximal(oracle):
    """With learning_rate = 1 the reference's rule coincides with FTRL-proximal
    (McMahan et al. 2013, alpha = 1): sigma = sqrt(n+g^2)-sqrt(n), z += g - sigma*w,
    w = -(z - sgn(z) l1) / (beta + sqrt(n) + l2) outside the l1 ball, else 0."""
    D = 6
    beta, l1, l2 = 1.0, 0.3, 0.7
    t = oracle.Table(oracle.FTRL, D, buckets=64, learning_rate=1.0, beta=beta, lambda1=l1, lambda2=l2)
    t.set_rows(SIGN, np.zeros((1, D), dtype=np.float32))
    rng = np.random.default_rng(3)
    w = np.zeros(D)
    z = np.zeros(D)
    n = np.zeros(D)
    for _ in range(25):
        g = (rng.standard_normal(D) * 0.4).astype(np.float32)
        t.push(one_info(oracle, 1), g[None, :])
        g64 = g.astype(np.float64)
        sigma = np.sqrt(n + g64 ** 2) - np.sqrt(n)
        z = z + g64 - sigma * w
        n = n + g64 ** 2
        w = np.where(np.abs(z) <= l1, 0.0, -(z - np.sign(z) * l1) / (beta + np.sqrt(n) + l2))
    ow, ost, _ = t.get_rows(SIGN)
    np.testing.assert_allclose(ow[0], w, rtol=2e-5, atol=1e-6)
    np.testing.assert_allclose(ost[0, :D], z, rtol=2e-5, atol=1e-6)


# ------------------------------------------------ table behaviour (A3/A4/A6)
def test_pull_returns_snapshot_rows_bit_exact(oracle):
    rng = np.random.default_rng(0)
    D = 8
    t = oracle.Table(oracle.ADAGRAD, D, buckets=1024, initial_g2sum=0.1)
    signs = rng.integers(0, 1 << 63, 500, dtype=np.uint64)
    w = rng.uniform(-0.01, 0.01, (500, D)).astype(np.float32)
    t.set_rows(signs, w)
    order = rng.permutation(500)[:300]
    out = t.pull(signs[order])
    assert (out.view(np.int32) == w[order].view(np.int32)).all()
    assert t.key_count() == len(np.unique(signs))


@pytest.mark.parametrize("kind,dim", [(0, 16), (1, 16), (2, 1), (0, 64)])
def test_new_rows_follow_the_initialiser(oracle, kind, dim):
    """N(0, 1/sqrt(dim)) * initial_scale; mean and std within 1 %, fresh state."""
    scale = 0.1
    t = oracle.Table(kind, dim, buckets=1 << 16, seed=5, initial_scale=scale, initial_g2sum=0.25)
    n = max(20000, 400000 // dim)
    signs = np.arange(1, n + 1, dtype=np.uint64)
    w = t.pull(signs)
    sigma = scale / np.sqrt(dim)
    assert abs(w.mean()) < 0.01 * sigma
    assert abs(w.std() / sigma - 1) < 0.01
    _, st, found = t.get_rows(signs[:10])
    assert found.all()
    if kind == 0:
        assert (st[:, 0] == np.float32(0.25)).all() and (st[:, 1:] == 0).all()
    else:
        assert (st == 0).all()


def test_zero_init_mode(oracle):
    t = oracle.Table(oracle.ADAM, 4, zero_init=True, buckets=64)
    assert (t.pull(np.asarray([1, 2, 3], dtype=np.uint64)) == 0).all()


def test_push_of_unknown_sign_is_reported(oracle):
    t = oracle.Table(oracle.ADAGRAD, 4, buckets=64)
    assert t.push(one_info(oracle, 1, sign=99), np.ones((1, 4), dtype=np.float32)) == 1


def test_same_sign_in_several_slots_is_applied_sequentially(oracle):
    """Slot-major sequential Applies (sparse_table_ops.cc:350-361, sparse_table.cc:72-82):
    equal to Apply(g0) then Apply(g1) then Apply(g2), different from one Apply of the sum."""
    D, lr = 4, 0.1
    hp = dict(learning_rate=lr, initial_g2sum=0.1, epsilon=1e-8)
    sign = np.int64(77)
    values = [np.asarray([sign, 5], dtype=np.int64), np.asarray([6, sign, sign], dtype=np.int64),
              np.asarray([sign], dtype=np.int64)]
    labels = [np.zeros_like(v) for v in values]
    grads = [np.full((2, D), 0.5, np.float32), np.full((2, D), -0.25, np.float32), np.full((1, D), 1.0, np.float32)]
    w0 = np.full((1, D), 0.5, dtype=np.float32)

    a = oracle.Table(oracle.ADAGRAD, D, buckets=64, **hp)
    for s in (5, 6, 77):
        a.set_rows(np.asarray([s], dtype=np.uint64), w0)
    rc, counts = a.push_op(values, grads, labels)
    assert rc == 0 and counts.tolist() == [2, 2, 1]

    b = oracle.Table(oracle.ADAGRAD, D, buckets=64, **hp)
    b.set_rows(np.asarray([77], dtype=np.uint64), w0)
    for g, show in ((grads[0][0], 1), (grads[1][1], 2), (grads[2][0], 1)):
        b.push(one_info(oracle, show, sign=77), g[None, :])
    wa, sa, _ = a.get_rows(np.asarray([77], dtype=np.uint64))
    wb, sb, _ = b.get_rows(np.asarray([77], dtype=np.uint64))
    assert (wa == wb).all() and (sa == sb).all()
    assert sa[0, 1] == 4.0  # show = 1 + 2 + 1

    c = oracle.Table(oracle.ADAGRAD, D, buckets=64, **hp)
    c.set_rows(np.asarray([77], dtype=np.uint64), w0)
    c.push(one_info(oracle, 4, sign=77), (grads[0][0] + grads[1][1] + grads[2][0])[None, :])
    wc, _, _ = c.get_rows(np.asarray([77], dtype=np.uint64))
    assert np.abs(wa - wc).max() > 1e-3


def test_pull_op_fills_variable_rows_and_leaves_the_rest(oracle):
    D = 4
    t = oracle.Table(oracle.ADAGRAD, D, buckets=64)
    signs = np.asarray([10, 20, 30], dtype=np.uint64)
    w = np.arange(12, dtype=np.float32).reshape(3, D)
    t.set_rows(signs, w)
    values = [np.asarray([20, 10, 20, 30], dtype=np.int64), np.asarray([30, 30], dtype=np.int64)]
    vars_ = [np.full((5, D), -1, np.float32), np.full((3, D), -1, np.float32)]
    rc, mapped, counts = t.pull_op(values, vars_)
    assert rc == 0 and counts.tolist() == [3, 1]
    assert mapped[0].tolist() == [0, 1, 0, 2] and mapped[1].tolist() == [0, 0]
    assert (vars_[0][:3] == w[[1, 0, 2]]).all() and (vars_[0][3:] == -1).all()
    assert (vars_[1][0] == w[2]).all() and (vars_[1][1:] == -1).all()
    # U_s must stay strictly below the variable's rows (CHECK_LT, sparse_table_ops.cc:136)
    rc, _, _ = t.pull_op([np.asarray([1, 2, 3], dtype=np.int64)], [np.zeros((3, D), np.float32)])
    assert rc == 4
