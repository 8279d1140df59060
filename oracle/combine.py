"""CPU oracle of the step TensorFlow runs around the pull / push ops of one
slot: the combiner of `embedding_lookup_sparse` after the pull and the
reduction of its gradient to one row per distinct id before the push.

TEST INFRASTRUCTURE (checker only), numpy.

The algorithm lives in TensorFlow (third party, pinned by the reference's
WORKSPACE:7-11 to v2.2.0, not in the reference tree), reached through
`tf.feature_column.embedding_column.get_dense_tensor`
(tensornet/layers/embedding_features.py:278-280) with the mapped ids of
tensornet/feature_column/category_column.py:42-51 as `sp_ids`.  Restated from
its published definition (tf.nn.embedding_lookup_sparse / safe_embedding_lookup_sparse,
no `sp_weights`):

  forward   out[b, :] = (sum over the lookups i of example b, in order, of params[ids[i], :]) / d(n_b)
            d(n) = 1 (sum), n (mean), sqrt(n) (sqrtn); an example without lookups gives zeros
  backward  d params[j, :] = sum over the lookups i with ids[i] == j, in order, of d out[b(i), :] * (1 / d(n_b(i)))
            delivered as IndexedSlices over unique(ids); mapped ids are first-occurrence ranks, so
            row j of the slices is the j-th distinct sign of the slot -- the `grads` input of
            SparseTablePush (core/kernels/sparse_table_ops.cc:336-352)

All sums run in float32 in occurrence order, as a single-threaded CPU kernel
would; the GPU path is compared within a tolerance.  No reference fixture holds
values for this step: parity unpinned by the reference, pinned in
tests/test_oracle_combine.py by brute force, closed forms and the adjoint
identity <A v, g> = <v, A^T g>.
"""
import numpy as np

SUM, MEAN, SQRTN = 0, 1, 2


def _norm(n, combiner):
    """Divisor of the forward pass per example (TF's SparseSegmentMean / SqrtN reductions
    divide the segment sum); 1 for examples without lookups."""
    n = np.asarray(n, dtype=np.float32)
    if combiner == SUM:
        return np.ones_like(n)
    n = np.maximum(n, np.float32(1))
    return n if combiner == MEAN else np.sqrt(n).astype(np.float32)


def combine_forward(ids, example, params, batch, combiner):
    """ids[i] in [0, rows), example[i] in [0, batch) non-decreasing; returns float32 [batch, dim]."""
    ids = np.asarray(ids, dtype=np.int64)
    example = np.asarray(example, dtype=np.int64)
    params = np.asarray(params, dtype=np.float32)
    out = np.zeros((batch, params.shape[1]), np.float32)
    np.add.at(out, example, params[ids])  # unbuffered: adds in occurrence order, float32
    counts = np.bincount(example, minlength=batch)
    return (out / _norm(counts, combiner)[:, None]).astype(np.float32)


def combine_backward(ids, example, dout, batch, combiner, rows):
    """Gradient rows for ids 0 .. rows-1 (float32 [rows, dim]) from dout [batch, dim]: every
    lookup contributes dout[example] * (1 / divisor of its example) (the scaling TF's
    SparseSegmentMeanGrad / SqrtNGrad apply), summed per id in occurrence order."""
    ids = np.asarray(ids, dtype=np.int64)
    example = np.asarray(example, dtype=np.int64)
    dout = np.asarray(dout, dtype=np.float32)
    counts = np.bincount(example, minlength=batch)
    scale = (np.float32(1) / _norm(counts, combiner)).astype(np.float32)
    g = np.zeros((rows, dout.shape[1]), np.float32)
    np.add.at(g, ids, dout[example] * scale[example][:, None])
    return g
