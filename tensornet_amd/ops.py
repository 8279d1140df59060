"""Operator surface of the hot path: the four TensorFlow ops of the reference
(core/ops/sparse_table_ops.cc:21-53, core/ops/dense_table_ops.cc:21-37, Python
wrappers tensornet/core/gen_sparse_table_ops.py / gen_dense_table_ops.py) with
the same names and argument order, taking torch tensors that live on the GPU.
Tensors are only used as device memory: every call goes through the C ABI with
raw device pointers and the current HIP stream.

A "resource" (tf.Variable handle in the reference) is here the variable's
torch tensor itself, updated in place.
"""
import ctypes as C

import torch

from . import _lib


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require(t, dtype, what):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError("%s must be a CUDA/HIP tensor" % what)
    if t.dtype != dtype:
        raise ValueError("%s must have dtype %s, got %s" % (what, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % what)


class BoundSparseTablePull:
    """SparseTablePull bound to fixed tensors, the way an op kernel of a built
    graph sees its inputs: arguments are validated and marshalled once, the
    mapped-id outputs allocated once; every call only crosses the C ABI (with the
    stream current at that moment).  Calling it returns the N mapped-id tensors."""

    def __init__(self, resources, values, table_handle):
        n = len(values)
        if len(resources) != n:
            raise ValueError("SparseTable pull num_inputs: %d not equal: %d" % (len(resources) + n, n * 2))
        if n == 0:
            raise ValueError("SparseTable pull needs at least one slot")
        dim = None
        for i in range(n):
            _require(resources[i], torch.float32, "resources[%d]" % i)
            _require(values[i], torch.int64, "values[%d]" % i)
            if resources[i].dim() != 2:
                raise ValueError(
                    "sparse pull variable must Matrix(sign_id_cnt, dim), saw: %s" % (tuple(resources[i].shape),)
                )
            if values[i].dim() != 1:
                raise ValueError("values[%d] must have rank 1" % i)
            if dim is None:
                dim = resources[i].shape[1]
            elif dim != resources[i].shape[1]:
                raise _lib.TensorNetError(3, "all variables of one pull must have the same dim")
        lens = [v.numel() for v in values]
        # one allocation for all mapped ids, handed out as per-slot views
        flat = torch.empty(sum(lens), dtype=torch.int64, device=values[0].device)
        self.mapped = list(flat.split(lens)) if sum(lens) > 0 else [torch.empty_like(v) for v in values]
        self._keep = (list(resources), list(values), flat)
        self._fn = _lib.load().tn_sparse_table_pull_op
        self._args = (
            table_handle,
            n,
            _lib.ptr_array([v.data_ptr() for v in values]),
            _lib.i64_array(lens),
            _lib.ptr_array([r.data_ptr() for r in resources]),
            _lib.i64_array([r.shape[0] for r in resources]),
            int(dim),
            _lib.ptr_array([m.data_ptr() for m in self.mapped]),
        )

    def __call__(self):
        _lib.check(self._fn(*self._args, _stream()))
        return self.mapped


class BoundSparseTablePush:
    """SparseTablePush bound to fixed tensors (see BoundSparseTablePull)."""

    def __init__(self, values, grads, feature_labels, table_handle):
        n = len(values)
        if len(grads) != n or len(feature_labels) != n:
            raise ValueError(
                "SparseTable push num_inputs: %d not equal: %d" % (n + len(grads) + len(feature_labels), n * 3)
            )
        if n == 0:
            raise ValueError("SparseTable push needs at least one slot")
        dim = None
        for i in range(n):
            _require(values[i], torch.int64, "values[%d]" % i)
            _require(grads[i], torch.float32, "grads[%d]" % i)
            _require(feature_labels[i], torch.int64, "feature_labels[%d]" % i)
            if grads[i].dim() != 2:
                raise ValueError("sparse push grad must Matrix(sign_id_cnt, dim), saw: %s" % (tuple(grads[i].shape),))
            if feature_labels[i].numel() != values[i].numel():
                raise ValueError("feature_labels[%d] must have one label per lookup" % i)
            if dim is None:
                dim = grads[i].shape[1]
            elif dim != grads[i].shape[1]:
                raise _lib.TensorNetError(3, "all gradients of one push must have the same dim")
        self._keep = (list(values), list(grads), list(feature_labels))
        self._fn = _lib.load().tn_sparse_table_push_op
        self._args = (
            table_handle,
            n,
            _lib.ptr_array([v.data_ptr() for v in values]),
            _lib.i64_array([v.numel() for v in values]),
            _lib.ptr_array([g.data_ptr() for g in grads]),
            _lib.i64_array([g.shape[0] for g in grads]),
            int(dim),
            _lib.ptr_array([l.data_ptr() for l in feature_labels]),
        )

    def __call__(self):
        _lib.check(self._fn(*self._args, _stream()))


def sparse_table_pull(resources, values, table_handle):
    """SparseTablePull.  resources: N float32 variables [rows, dim] (updated in
    place: row j <- embedding of the j-th distinct sign of the slot);
    values: N int64 rank-1 tensors of signs.  Returns N int64 tensors of mapped
    ids (same shapes as values)."""
    return BoundSparseTablePull(resources, values, table_handle)()


def sparse_table_push(values, grads, feature_labels, table_handle):
    """SparseTablePush.  grads[i] is [U_i, dim] with row j the gradient of the
    j-th distinct sign of values[i]; feature_labels[i] has one int64 label per
    lookup.  Returns nothing (the update is enqueued on the current stream)."""
    BoundSparseTablePush(values, grads, feature_labels, table_handle)()


COMBINERS = {"sum": 0, "mean": 1, "sqrtn": 2}


def _combiner(combiner):
    if combiner not in COMBINERS:
        raise ValueError("combiner must be one of 'sum', 'mean', 'sqrtn', got %r" % (combiner,))
    return COMBINERS[combiner]


def embedding_lookup_sparse(resources, mapped_values, example_ids, batch_size, table_handle, combiner="mean"):
    """What TensorFlow does with the pull's results for every slot
    (tf.nn.embedding_lookup_sparse behind embedding_column.get_dense_tensor,
    tensornet/layers/embedding_features.py:278-280): out[s][b] = combiner over
    the rows resources[s][mapped_values[s][i]] of the lookups i of example b.
    example_ids[s][i] is the example of lookup i (SparseTensor.indices[:, 0]).
    Returns N float32 tensors [batch_size, dim]."""
    return BoundEmbeddingLookupSparse(resources, mapped_values, example_ids, batch_size, table_handle, combiner)()


class BoundEmbeddingLookupSparse:
    """embedding_lookup_sparse bound to fixed tensors (see BoundSparseTablePull): the variables and mapped ids of a
    bound pull, the example ids, and outputs allocated once.  Calling it returns the N [batch_size, dim] tensors."""

    def __init__(self, resources, mapped_values, example_ids, batch_size, table_handle, combiner="mean"):
        n = len(mapped_values)
        if len(resources) != n or len(example_ids) != n or n == 0:
            raise ValueError("embedding_lookup_sparse needs one variable, id tensor and example-id tensor per slot")
        for i in range(n):
            _require(resources[i], torch.float32, "resources[%d]" % i)
            _require(mapped_values[i], torch.int64, "mapped_values[%d]" % i)
            _require(example_ids[i], torch.int64, "example_ids[%d]" % i)
            if example_ids[i].numel() != mapped_values[i].numel():
                raise ValueError("example_ids[%d] must have one entry per lookup" % i)
        dim = resources[0].shape[1]
        flat = torch.empty((n, batch_size, dim), dtype=torch.float32, device=resources[0].device)
        self.out = list(flat.unbind(0))
        self._keep = (list(resources), list(mapped_values), list(example_ids), flat)
        self._fn = _lib.load().tn_sparse_table_combine_op
        self._args = (
            table_handle,
            n,
            _lib.ptr_array([v.data_ptr() for v in mapped_values]),
            _lib.i64_array([v.numel() for v in mapped_values]),
            _lib.ptr_array([e.data_ptr() for e in example_ids]),
            _lib.ptr_array([r.data_ptr() for r in resources]),
            _lib.i64_array([r.shape[0] for r in resources]),
            int(dim),
            int(batch_size),
            _combiner(combiner),
            _lib.ptr_array([o.data_ptr() for o in self.out]),
        )

    def __call__(self):
        _lib.check(self._fn(*self._args, _stream()))
        return self.out


class BoundSparseTablePushPooled:
    """SparseTablePush fed with the gradients of the combiner's outputs
    (pooled_grads[s]: [batch_size, dim]) instead of per-distinct-sign rows; the
    reduction TensorFlow performs in between (gradient of embedding_lookup_sparse
    summed per distinct id) runs on the device.  Bound to fixed tensors like
    BoundSparseTablePush."""

    def __init__(self, values, example_ids, pooled_grads, feature_labels, table_handle, combiner="mean"):
        n = len(values)
        if len(example_ids) != n or len(pooled_grads) != n or len(feature_labels) != n or n == 0:
            raise ValueError("SparseTable push (pooled) needs values, example ids, gradients and labels per slot")
        for i in range(n):
            _require(values[i], torch.int64, "values[%d]" % i)
            _require(example_ids[i], torch.int64, "example_ids[%d]" % i)
            _require(pooled_grads[i], torch.float32, "pooled_grads[%d]" % i)
            _require(feature_labels[i], torch.int64, "feature_labels[%d]" % i)
            if pooled_grads[i].dim() != 2 or pooled_grads[i].shape != pooled_grads[0].shape:
                raise ValueError("pooled_grads must all be Matrix(batch_size, dim)")
            if example_ids[i].numel() != values[i].numel() or feature_labels[i].numel() != values[i].numel():
                raise ValueError("example_ids / feature_labels of slot %d must have one entry per lookup" % i)
        self._keep = (list(values), list(example_ids), list(pooled_grads), list(feature_labels))
        self._fn = _lib.load().tn_sparse_table_push_pooled_op
        self._args = (
            table_handle,
            n,
            _lib.ptr_array([v.data_ptr() for v in values]),
            _lib.i64_array([v.numel() for v in values]),
            _lib.ptr_array([e.data_ptr() for e in example_ids]),
            _lib.ptr_array([g.data_ptr() for g in pooled_grads]),
            int(pooled_grads[0].shape[0]),
            int(pooled_grads[0].shape[1]),
            _combiner(combiner),
            _lib.ptr_array([l.data_ptr() for l in feature_labels]),
        )

    def __call__(self):
        _lib.check(self._fn(*self._args, _stream()))


def sparse_table_push_pooled(values, example_ids, pooled_grads, feature_labels, table_handle, combiner="mean"):
    BoundSparseTablePushPooled(values, example_ids, pooled_grads, feature_labels, table_handle, combiner)()


def sparse_table_sync(table_handle):
    """Waits for enqueued pushes of the table and raises their latched error."""
    _lib.check(_lib.load().tn_sparse_table_sync(table_handle))


def sparse_table_last_unique_counts(table_handle, n_slots):
    out = (C.c_int64 * n_slots)()
    _lib.check(_lib.load().tn_sparse_table_last_unique_counts(table_handle, n_slots, out))
    return [int(x) for x in out]


def dense_table_init(vars, table_handle):
    """DenseTableInit: the table takes the concatenation of the variables."""
    for i, v in enumerate(vars):
        _require(v, torch.float32, "vars[%d]" % i)
    rc = _lib.load().tn_dense_table_init(
        table_handle,
        len(vars),
        _lib.ptr_array([v.data_ptr() for v in vars]),
        _lib.i64_array([v.numel() for v in vars]),
        _stream(),
    )
    _lib.check(rc)


def dense_table_push_pull(vars, grads, learning_rate, table_handle):
    """DenseTablePushPull: optimizer step with the concatenated gradients, new
    weights written back into the variables (in place)."""
    if len(vars) != len(grads):
        raise ValueError("DenseTable pushpull num_inputs: %d not equal: %d" % (len(vars) + len(grads) + 1, 2 * len(vars) + 1))
    for i, (v, g) in enumerate(zip(vars, grads)):
        _require(v, torch.float32, "vars[%d]" % i)
        _require(g, torch.float32, "grads[%d]" % i)
        if v.numel() != g.numel():
            raise ValueError(
                "DenseTable var tensor length: %d not equal grad tensor length: %d" % (v.numel(), g.numel())
            )
    rc = _lib.load().tn_dense_table_push_pull(
        table_handle,
        len(vars),
        _lib.ptr_array([v.data_ptr() for v in vars]),
        _lib.ptr_array([g.data_ptr() for g in grads]),
        _lib.i64_array([g.numel() for g in grads]),
        float(learning_rate),
        _stream(),
    )
    _lib.check(rc)


# ------------------------------------------------------------ table level
def table_pull(table_handle, signs, dim):
    """SparseTable::Pull: signs int64/uint64-as-int64 [n] -> float32 [n, dim]."""
    _require(signs, torch.int64, "signs")
    out = torch.empty((signs.numel(), dim), dtype=torch.float32, device=signs.device)
    rc = _lib.load().tn_sparse_table_pull(table_handle, signs.data_ptr(), signs.numel(), dim, out.data_ptr(), _stream())
    _lib.check(rc)
    return out


def table_push(table_handle, sign_infos, grads):
    """SparseTable::Push: sign_infos is an int64 tensor [n, 2] holding the 16-byte
    records (sign, batch_show | batch_click << 32); grads float32 [n, dim]."""
    _require(sign_infos, torch.int64, "sign_infos")
    _require(grads, torch.float32, "grads")
    n = grads.shape[0]
    rc = _lib.load().tn_sparse_table_push(
        table_handle, sign_infos.data_ptr(), grads.data_ptr(), n, grads.shape[1], _stream()
    )
    _lib.check(rc)


def make_sign_infos(signs, shows, clicks):
    """Packs int64 signs and int32-valued shows/clicks into 16-byte records."""
    rec = torch.empty((signs.numel(), 2), dtype=torch.int64, device=signs.device)
    rec[:, 0] = signs
    rec[:, 1] = (shows.to(torch.int64) & 0xFFFFFFFF) | (clicks.to(torch.int64) << 32)
    return rec


def table_load_rows(table_handle, signs, w, state=None):
    _require(signs, torch.int64, "signs")
    _require(w, torch.float32, "w")
    if state is not None:
        _require(state, torch.float32, "state")
    rc = _lib.load().tn_sparse_table_load_rows(
        table_handle,
        signs.data_ptr(),
        w.data_ptr(),
        state.data_ptr() if state is not None else None,
        signs.numel(),
        _stream(),
    )
    _lib.check(rc)


def table_export_rows(table_handle, signs):
    from .core import sparse_table_row_layout

    _require(signs, torch.int64, "signs")
    wf, sf = sparse_table_row_layout(table_handle)
    n = signs.numel()
    w = torch.empty((n, wf), dtype=torch.float32, device=signs.device)
    st = torch.empty((n, sf), dtype=torch.float32, device=signs.device)
    found = torch.empty((n,), dtype=torch.uint8, device=signs.device)
    rc = _lib.load().tn_sparse_table_export_rows(
        table_handle, signs.data_ptr(), n, w.data_ptr(), st.data_ptr(), found.data_ptr(), _stream()
    )
    _lib.check(rc)
    return w, st, found


def table_delete_by_show(table_handle, signs):
    """Value::DeleteByShow for the rows of `signs` (uint8 tensor: 1 = the row would be left out of
    a saved table, 0 = kept or absent)."""
    _require(signs, torch.int64, "signs")
    out = torch.empty((signs.numel(),), dtype=torch.uint8, device=signs.device)
    _lib.check(_lib.load().tn_sparse_table_delete_by_show(table_handle, signs.data_ptr(), signs.numel(),
                                                          out.data_ptr(), _stream()))
    return out


def dense_table_range(table_handle):
    """(begin, end) of the table's elements this shard holds (optimizer_kernel.h:55-57)."""
    b, e = C.c_int64(), C.c_int64()
    _lib.check(_lib.load().tn_dense_table_range(table_handle, C.byref(b), C.byref(e)))
    return b.value, e.value


def dense_table_get_weight(table_handle, device="cuda"):
    b, e = dense_table_range(table_handle)
    w = torch.empty((e - b,), dtype=torch.float32, device=device)
    _lib.check(_lib.load().tn_dense_table_get_weight(table_handle, w.data_ptr(), _stream()))
    return w


def dense_table_get_state(table_handle, n_states=2, device="cuda"):
    b, e = dense_table_range(table_handle)
    outs = [torch.empty((e - b,), dtype=torch.float32, device=device) for _ in range(n_states)]
    ptrs = [o.data_ptr() for o in outs] + [None] * (3 - n_states)
    _lib.check(_lib.load().tn_dense_table_get_state(table_handle, ptrs[0], ptrs[1], ptrs[2], _stream()))
    return outs
