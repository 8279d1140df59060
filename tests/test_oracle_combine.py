"""Pins oracle/combine.py (the combiner TensorFlow runs around the pull / push
ops) against what the mathematics fixes: an element-by-element restatement,
closed forms, and the adjoint identity between forward and backward."""
import numpy as np
import pytest

from oracle import combine as C


def brute_forward(ids, example, params, batch, combiner):
    out = [[0.0] * params.shape[1] for _ in range(batch)]
    cnt = [0] * batch
    for i, b in zip(ids, example):
        cnt[b] += 1
        for c in range(params.shape[1]):
            out[b][c] = float(np.float32(out[b][c]) + params[i, c])
    for b in range(batch):
        if cnt[b] and combiner != C.SUM:
            d = np.float32(cnt[b]) if combiner == C.MEAN else np.sqrt(np.float32(cnt[b]))
            out[b] = [float(np.float32(v) / d) for v in out[b]]
    return np.asarray(out, np.float32)


def brute_backward(ids, example, dout, batch, combiner, rows):
    cnt = np.bincount(example, minlength=batch)
    g = np.zeros((rows, dout.shape[1]), np.float32)
    for i, b in zip(ids, example):
        if combiner == C.SUM:
            s = np.float32(1)
        elif combiner == C.MEAN:
            s = np.float32(1) / np.float32(cnt[b])
        else:
            s = np.float32(1) / np.sqrt(np.float32(cnt[b]))
        g[i] = g[i] + dout[b] * s
    return g


def random_case(rng, batch=13, rows=9, dim=5, lookups=40):
    example = np.sort(rng.integers(0, batch, lookups))
    ids = rng.integers(0, rows, lookups)
    params = rng.standard_normal((rows, dim)).astype(np.float32)
    dout = rng.standard_normal((batch, dim)).astype(np.float32)
    return ids, example, params, dout


@pytest.mark.parametrize("combiner", [C.SUM, C.MEAN, C.SQRTN])
def test_matches_the_element_by_element_restatement(combiner):
    rng = np.random.default_rng(combiner)
    for _ in range(5):
        ids, example, params, dout = random_case(rng)
        f = C.combine_forward(ids, example, params, 13, combiner)
        assert (f.view(np.int32) == brute_forward(ids, example, params, 13, combiner).view(np.int32)).all()
        g = C.combine_backward(ids, example, dout, 13, combiner, 9)
        assert (g.view(np.int32) == brute_backward(ids, example, dout, 13, combiner, 9).view(np.int32)).all()


def test_known_answers():
    ids = np.array([0, 1, 0, 2])
    example = np.array([0, 0, 2, 2])          # example 1 has no lookup
    params = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    assert C.combine_forward(ids, example, params, 3, C.SUM).tolist() == [[4, 6], [0, 0], [6, 8]]
    assert C.combine_forward(ids, example, params, 3, C.MEAN).tolist() == [[2, 3], [0, 0], [3, 4]]
    dout = np.array([[2, 4], [100, 100], [8, 16]], np.float32)
    # id 0 is looked up by examples 0 and 2, ids 1 and 2 once each; example 1 contributes nothing
    assert C.combine_backward(ids, example, dout, 3, C.SUM, 3).tolist() == [[10, 20], [2, 4], [8, 16]]
    assert C.combine_backward(ids, example, dout, 3, C.MEAN, 3).tolist() == [[5, 10], [1, 2], [4, 8]]
    four = np.array([0, 0, 0, 0])
    assert C.combine_forward(four, four, params, 1, C.SQRTN).tolist() == [[2, 4]]      # 4 * row0 / sqrt(4)
    assert C.combine_backward(four, four, dout[:1], 1, C.SQRTN, 1).tolist() == [[4, 8]]  # 4 * dout / 2


def test_closed_forms():
    rng = np.random.default_rng(7)
    ids, example, params, _ = random_case(rng, batch=6, rows=4, dim=3, lookups=30)
    ones = np.ones_like(params)
    counts = np.bincount(example, minlength=6).astype(np.float32)
    assert (C.combine_forward(ids, example, ones, 6, C.SUM) == counts[:, None]).all()
    assert (C.combine_forward(ids, example, ones, 6, C.MEAN) == (counts > 0)[:, None]).all()
    # the mean of identical rows is the row
    same = np.zeros(30, np.int64) + 2
    np.testing.assert_allclose(C.combine_forward(same, example, params, 6, C.MEAN)[counts > 0],
                               np.broadcast_to(params[2], (int((counts > 0).sum()), 3)), rtol=1e-6)
    # with every id distinct the backward pass is a gather of scaled rows
    uniq = np.arange(30)
    dout = rng.standard_normal((6, 3)).astype(np.float32)
    g = C.combine_backward(uniq, example, dout, 6, C.MEAN, 30)
    np.testing.assert_allclose(g, dout[example] / counts[example][:, None], rtol=1e-6)


@pytest.mark.parametrize("combiner", [C.SUM, C.MEAN, C.SQRTN])
def test_backward_is_the_adjoint_of_forward(combiner):
    """<A v, g> == <v, A^T g>; exact on small integers with power-of-two example sizes."""
    rng = np.random.default_rng(11 + combiner)
    sizes = rng.choice([1, 4, 16], 12)
    example = np.repeat(np.arange(12), sizes)
    ids = rng.integers(0, 10, len(example))
    params = rng.integers(-8, 9, (10, 4)).astype(np.float32)
    dout = rng.integers(-8, 9, (12, 4)).astype(np.float32)
    lhs = (C.combine_forward(ids, example, params, 12, combiner).astype(np.float64) * dout).sum()
    rhs = (params.astype(np.float64) * C.combine_backward(ids, example, dout, 12, combiner, 10)).sum()
    assert lhs == rhs
