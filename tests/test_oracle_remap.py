"""Pins the oracle's key remap (rows A1 / A5 of the hot path) without the
reference: hand-made known answers, an O(n^2) brute force, and the identity
with numpy.unique re-ranked by first index."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def brute_force(values):
    """mapped[i] = number of distinct signs whose first occurrence is before
    the first occurrence of values[i]."""
    values = [int(v) & 0xFFFFFFFFFFFFFFFF for v in values]
    mapped, signs = [], []
    for v in values:
        if v not in signs:
            signs.append(v)
        mapped.append(signs.index(v))
    return mapped, signs


def via_numpy_unique(values):
    u = np.asarray(values, dtype=np.int64).view(np.uint64)
    uniq, first, inverse = np.unique(u, return_index=True, return_inverse=True)
    order = np.argsort(first, kind="stable")
    rank = np.empty(len(uniq), dtype=np.int64)
    rank[order] = np.arange(len(uniq))
    return rank[inverse], uniq[order]


def test_known_answers(oracle):
    with open(os.path.join(HERE, "golden", "remap_kat.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        values = np.asarray(c["values"], dtype=np.int64)
        labels = np.asarray(c["labels"], dtype=np.int64)
        mapped, signs = oracle.pull_remap(values)
        assert mapped.tolist() == c["mapped"]
        assert [int(s) for s in signs] == c["signs"]
        infos = oracle.push_remap(values, labels)
        assert [int(s) for s in infos["sign"]] == c["signs"]
        assert infos["batch_show"].tolist() == c["show"]
        assert infos["batch_click"].tolist() == c["click"]


@pytest.mark.parametrize("seed", range(6))
def test_brute_force_and_unique(oracle, seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 400))
    vocab = int(rng.integers(1, 60))
    pool = rng.integers(-(1 << 63), (1 << 63) - 1, vocab, dtype=np.int64)
    values = pool[rng.integers(0, vocab, n)]
    labels = rng.integers(0, 3, n).astype(np.int64)
    mapped, signs = oracle.pull_remap(values)
    bm, bs = brute_force(values)
    assert mapped.tolist() == bm
    assert [int(s) for s in signs] == bs
    um, us = via_numpy_unique(values)
    assert (mapped == um).all() and (signs == us).all()
    # properties: equal signs <=> equal ids; first occurrences count 0,1,2,...
    assert (values[:, None] == values[None, :]).tolist() == (mapped[:, None] == mapped[None, :]).tolist()
    firsts = [mapped[i] for i in range(n) if mapped[i] not in mapped[:i]]
    assert firsts == list(range(len(signs)))
    infos = oracle.push_remap(values, labels)
    assert (infos["sign"] == signs).all()
    assert infos["batch_show"].sum() == n
    assert infos["batch_click"].sum() == labels.sum()
    for j, s in enumerate(signs):
        sel = values.view(np.uint64) == s
        assert infos["batch_show"][j] == sel.sum()
        assert infos["batch_click"][j] == labels[sel].sum()


def test_labels_are_narrowed_to_int(oracle):
    # static_cast<int>(fea_label_vec[i]), sparse_table_ops.cc:286
    values = np.asarray([1, 1], dtype=np.int64)
    labels = np.asarray([(1 << 32) + 5, 2], dtype=np.int64)
    infos = oracle.push_remap(values, labels)
    assert infos["batch_click"].tolist() == [7]
