"""Pins the oracle's dense update (rows A8 / A9).  The arithmetic of the
reference lives in Eigen (a third-party dependency that is not in the
reference tree): elementwise float + - * / sqrt, correctly rounded per
element, double scalars narrowed to float.  Pinned by the scalar closed form
in numpy, by torch.optim.Adam (same rule when epsilon = 0), and by the
beta = 0 reduction."""
import numpy as np
import pytest
import torch

f32 = np.float32


def np_dense_adam(w, m, v, g, lr, b1, b2, eps, b1p, b2p):
    """adam_kernel.cc:46-55."""
    b1p = f32(b1p * f32(b1))
    b2p = f32(b2p * f32(b2))
    alpha = f32(np.float64(f32(lr)) * np.sqrt(1.0 - np.float64(b2p)) / (1.0 - np.float64(b1p)))
    c1 = f32(1.0 - np.float64(f32(b1)))
    c2 = f32(1.0 - np.float64(f32(b2)))
    m = (m + (g - m) * c1).astype(np.float32)
    v = (v + (g * g - v) * c2).astype(np.float32)
    w = (w - (m * alpha) / (np.sqrt(v, dtype=np.float32) + f32(eps))).astype(np.float32)
    return w, m, v, b1p, b2p


@pytest.mark.parametrize("total", [1, 7, 8, 1001, 4096])
def test_dense_adam_matches_numpy_closed_form(oracle, total):
    rng = np.random.default_rng(total)
    hp = dict(learning_rate=0.0, beta1=0.9, beta2=0.999, epsilon=1e-8)
    d = oracle.Dense(oracle.ADAM, total, **hp)
    assert d.num_blocks() == min(8, total) or d.num_blocks() == int(np.ceil(total / np.ceil(total / 8)))
    w = rng.uniform(-0.05, 0.05, total).astype(np.float32)
    d.set_weight(w)
    m = np.zeros(total, np.float32)
    v = np.zeros(total, np.float32)
    b1p = b2p = f32(1)
    for step in range(6):
        g = (rng.standard_normal(total) * 1e-4).astype(np.float32)
        lr = 1e-3 * (1 + step)  # the learning rate is an input of every step
        d.apply(g, lr)
        w, m, v, b1p, b2p = np_dense_adam(w, m, v, g, lr, 0.9, 0.999, 1e-8, b1p, b2p)
        assert (d.get_weight() == w).all()
        assert (d.get_state(0) == m).all() and (d.get_state(1) == v).all()


def test_dense_adam_equals_torch_adam_when_eps_is_zero(oracle):
    total, lr = 513, 1e-3
    rng = np.random.default_rng(1)
    w0 = rng.uniform(-0.05, 0.05, total).astype(np.float32)
    d = oracle.Dense(oracle.ADAM, total, beta1=0.9, beta2=0.999, epsilon=0.0)
    d.set_weight(w0)
    p = torch.nn.Parameter(torch.tensor(w0, dtype=torch.float64))
    opt = torch.optim.Adam([p], lr=lr, betas=(float(f32(0.9)), float(f32(0.999))), eps=0.0)
    for _ in range(20):
        g = (rng.standard_normal(total) * 1e-2).astype(np.float32)
        g[g == 0] = 1e-3
        d.apply(g, lr)
        p.grad = torch.tensor(g, dtype=torch.float64)
        opt.step()
    np.testing.assert_allclose(d.get_weight(), p.detach().numpy(), rtol=1e-5, atol=1e-7)


def test_dense_adam_beta_zero_reduces_to_normalised_step(oracle):
    """beta1 = beta2 = 0: alpha = lr, m = g, v = g^2, w -= lr*g/(|g| + eps)."""
    total, lr, eps = 64, 0.25, 0.5
    d = oracle.Dense(oracle.ADAM, total, beta1=0.0, beta2=0.0, epsilon=eps)
    w0 = np.linspace(-1, 1, total).astype(np.float32)
    g = np.linspace(-2, 2, total).astype(np.float32)
    d.set_weight(w0)
    d.apply(g, lr)
    expect = w0 - (g * f32(lr)) / (np.abs(g) + f32(eps))
    np.testing.assert_array_equal(d.get_weight(), expect.astype(np.float32))


def test_dense_adagrad_closed_form(oracle):
    """ada_grad_kernel.cc:42-48 with mom_decay_rate = 0 (m = g) and
    grad_decay_rate = 1: after t steps w -= lr*g/(sqrt(g2sum0 + sum g^2)/sqrt(t) + eps)."""
    total, lr, eps = 100, 0.1, 1e-3
    rng = np.random.default_rng(2)
    d = oracle.Dense(oracle.ADAGRAD, total, initial_g2sum=0.5, epsilon=eps, grad_decay_rate=1.0, mom_decay_rate=0.0)
    w = rng.uniform(-1, 1, total)
    d.set_weight(w.astype(np.float32))
    w = w.astype(np.float32).astype(np.float64)
    g2 = np.full(total, 0.5)
    for t in range(1, 6):
        g = rng.standard_normal(total).astype(np.float32)
        d.apply(g, lr)
        g2 += g.astype(np.float64) ** 2
        w -= lr * g / (np.sqrt(g2) / np.sqrt(t) + eps)
    np.testing.assert_allclose(d.get_weight(), w, rtol=1e-5, atol=1e-6)
    # default mom_decay_rate = 1 freezes the weights: m += (g - m) * 0
    d2 = oracle.Dense(oracle.ADAGRAD, 8)
    d2.set_weight(np.ones(8, np.float32))
    d2.apply(np.ones(8, np.float32), 1.0)
    assert (d2.get_weight() == 1).all()
