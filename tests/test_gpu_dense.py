"""GPU parity of the DenseTable update against the CPU oracle (tolerance 1e-5
relative / 1e-7 absolute on weights and moments)."""
import numpy as np
import pytest
import torch

from helpers import ATOL, RTOL, dev

pytestmark = pytest.mark.gpu


def split(total, sizes):
    out, off = [], 0
    for n in sizes:
        out.append((off, off + n))
        off += n
    assert off == total
    return out


@pytest.mark.parametrize("sizes", [[1], [7, 1, 8], [1000, 24, 4096, 3, 77], [64 * 64, 64, 64 * 32, 32]])
def test_dense_adam_push_pull(tn, oracle, sizes):
    total = sum(sizes)
    rng = np.random.default_rng(total)
    hp = dict(beta1=0.9, beta2=0.999, epsilon=1e-8)
    h = tn.core.create_dense_table(tn.core.Adam(learning_rate=1e-3, **hp))
    d = oracle.Dense(oracle.ADAM, total, **hp)
    w0 = rng.uniform(-0.05, 0.05, total).astype(np.float32)
    d.set_weight(w0)
    vars_ = [dev(w0[a:b]) for a, b in split(total, sizes)]
    tn.ops.dense_table_init(vars_, h)
    for step in range(5):
        g = (rng.standard_normal(total) * 1e-4).astype(np.float32)
        lr = 1e-3 * (step + 1)
        d.apply(g, lr)
        tn.ops.dense_table_push_pull(vars_, [dev(g[a:b]) for a, b in split(total, sizes)], lr, h)
        got = torch.cat(vars_).cpu().numpy()
        np.testing.assert_allclose(got, d.get_weight(), rtol=RTOL, atol=ATOL)
    assert torch.equal(tn.ops.dense_table_get_weight(h), torch.cat(vars_))
    m, v = tn.ops.dense_table_get_state(h, 2)
    np.testing.assert_allclose(m.cpu().numpy(), d.get_state(0), rtol=RTOL, atol=1e-12)
    np.testing.assert_allclose(v.cpu().numpy(), d.get_state(1), rtol=RTOL, atol=1e-15)
    same = (torch.cat(vars_).cpu().numpy() == d.get_weight()).mean()
    assert same > 0.99


@pytest.mark.parametrize("sizes", [[5000], [7, 1, 8], [1000, 24, 4099, 3, 77]])
def test_dense_adagrad_push_pull(tn, oracle, sizes):
    """Aligned bodies go through the 16-byte kernel, odd offsets and tails through the scalar one."""
    total = sum(sizes)
    rng = np.random.default_rng(4)
    hp = dict(initial_g2sum=0.5, epsilon=1e-3, grad_decay_rate=0.9, mom_decay_rate=0.5)
    h = tn.core.create_dense_table(tn.core.AdaGrad(**hp))
    d = oracle.Dense(oracle.ADAGRAD, total, **hp)
    w0 = rng.uniform(-1, 1, total).astype(np.float32)
    d.set_weight(w0)
    vars_ = [dev(w0[a:b]) for a, b in split(total, sizes)]
    tn.ops.dense_table_init(vars_, h)
    for _ in range(4):
        g = rng.standard_normal(total).astype(np.float32)
        d.apply(g, 0.1)
        tn.ops.dense_table_push_pull(vars_, [dev(g[a:b]) for a, b in split(total, sizes)], 0.1, h)
    np.testing.assert_allclose(torch.cat(vars_).cpu().numpy(), d.get_weight(), rtol=RTOL, atol=ATOL)
    assert torch.equal(tn.ops.dense_table_get_weight(h), torch.cat(vars_))


def test_dense_errors(tn):
    h = tn.core.create_dense_table(tn.core.Adam())
    g = torch.zeros(16, device="cuda")
    with pytest.raises(tn.TensorNetError) as e:  # push before init
        tn.ops.dense_table_push_pull([g.clone()], [g], 0.1, h)
    assert e.value.code == 9
    tn.ops.dense_table_init([g.clone()], h)
    tn.ops.dense_table_init([g.clone()], h)  # same size again is fine (dense_table.cc:38-44)
    with pytest.raises(tn.TensorNetError) as e:
        tn.ops.dense_table_init([torch.zeros(17, device="cuda")], h)
    assert e.value.code == 8
    with pytest.raises(tn.TensorNetError) as e:  # CHECK_EQ(total_elements, TotalElements())
        tn.ops.dense_table_push_pull([torch.zeros(8, device="cuda")], [torch.zeros(8, device="cuda")], 0.1, h)
    assert e.value.code == 3
    with pytest.raises(tn.TensorNetError):
        tn.core.create_dense_table(tn.core.Ftrl())
    with pytest.raises(tn.TensorNetError):
        tn.core.create_dense_table(tn.core.Adam(), 2, 2)  # shard id outside the shard count


def test_dense_full_size_properties(tn):
    """2e8 parameters (cfg5's dense part): a step with g = 0 keeps w; a step from
    fresh moments moves every weight by -lr*sign(g) up to epsilon effects."""
    total = 2 * 10 ** 8
    h = tn.core.create_dense_table(tn.core.Adam(beta1=0.9, beta2=0.999, epsilon=1e-8))
    w = (torch.rand(total, device="cuda") - 0.5) * 0.1
    w0 = w.clone()
    tn.ops.dense_table_init([w], h)
    g = torch.randn(total, device="cuda") * 1e-4
    tn.ops.dense_table_push_pull([w], [g], 1e-3, h)
    # first step of Adam: m/(1-b1) = g, sqrt(v/(1-b2)) = |g| -> step = lr * g/(|g| + eps')
    step = w0 - w
    expect = 1e-3 * g / (g.abs() + 1e-8 / (1 - 0.999) ** 0.5)
    assert float((step - expect).abs().max()) < 2e-8
    del w0, step, expect
    w1 = w.clone()
    tn.ops.dense_table_push_pull([w], [torch.zeros_like(g)], 0.0, h)
    assert torch.equal(w, w1)
