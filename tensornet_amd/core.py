"""Configuration surface of the hot path, mirroring the reference's
`tensornet.core` (pybind module `_pywrap_tn`, core/main/py_wrapper.cc:61-263):
optimizer factories taking keyword arguments with the reference's names and
defaults, and table factories returning integer handles.
"""
import ctypes as C

from . import _lib


class _Opt(object):
    """Opaque optimizer object (the reference returns a PyCapsule)."""

    def __init__(self, handle, name):
        self.handle = handle
        self.name = name

    def __repr__(self):
        return "<tensornet_amd %s optimizer #%d>" % (self.name, self.handle)


def _fill(params, kwargs, allowed):
    for key, value in kwargs.items():
        if key not in allowed:
            # PYDICT_PARSE_KWARGS ignores unknown names (py_wrapper.cc:38-45)
            continue
        if key in ("no_show_days", "elimination_logic"):
            setattr(params, key, int(value))
        else:
            setattr(params, key, float(value))


def AdaGrad(**kwargs):
    """py_wrapper.cc:82-116.  learning_rate must be a float here (schedules
    are only evaluated for the dense path in the reference)."""
    lib = _lib.load()
    p = _lib.AdaGradParams()
    lib.tn_adagrad_params_default(C.byref(p))
    _fill(p, kwargs, [f for f, _ in _lib.AdaGradParams._fields_])
    if p.elimination_logic not in (0, 1):
        raise ValueError(
            "elimination_logic must be in the set of valid values {0, 1}, but got: %d" % p.elimination_logic
        )
    h = C.c_int32()
    _lib.check(lib.tn_opt_create_adagrad(C.byref(p), C.byref(h)))
    return _Opt(h.value, "AdaGrad")


def Adam(**kwargs):
    """py_wrapper.cc:117-133."""
    lib = _lib.load()
    p = _lib.AdamParams()
    lib.tn_adam_params_default(C.byref(p))
    _fill(p, kwargs, [f for f, _ in _lib.AdamParams._fields_])
    h = C.c_int32()
    _lib.check(lib.tn_opt_create_adam(C.byref(p), C.byref(h)))
    return _Opt(h.value, "Adam")


def Ftrl(**kwargs):
    """py_wrapper.cc:146-162."""
    lib = _lib.load()
    p = _lib.FtrlParams()
    lib.tn_ftrl_params_default(C.byref(p))
    _fill(p, kwargs, [f for f, _ in _lib.FtrlParams._fields_])
    h = C.c_int32()
    _lib.check(lib.tn_opt_create_ftrl(C.byref(p), C.byref(h)))
    return _Opt(h.value, "Ftrl")


def get_opt_learning_rate(opt):
    """py_wrapper.cc:134-145 (constant learning rate)."""
    lr = C.c_float()
    _lib.check(_lib.load().tn_opt_get_learning_rate(opt.handle, C.byref(lr)))
    return lr.value


def set_sparse_init_mode(opt, is_training):
    """py_wrapper.cc:163-168: zero-initialise new rows when not training."""
    _lib.check(_lib.load().tn_opt_set_sparse_zero_init(opt.handle, 0 if is_training else 1))


def create_sparse_table(opt, name, dimension, use_cvm=False, embedding_group=""):
    """py_wrapper.cc:169-181 -> CreateSparseTable (sparse_table.cc:169-186)."""
    h = C.c_uint32()
    _lib.check(
        _lib.load().tn_sparse_table_create(
            opt.handle,
            (name or "").encode(),
            int(dimension),
            1 if use_cvm else 0,
            1,
            0,
            (embedding_group or "").encode(),
            C.byref(h),
        )
    )
    return h.value


def create_dense_table(opt, shard_num=1, self_shard_id=0):
    """py_wrapper.cc:182-191 -> CreateDenseTable (dense_table.cc:180-186).  The reference takes
    the shard count and id from its cluster (RankNum, Rank); one worker is the default here."""
    h = C.c_uint32()
    _lib.check(_lib.load().tn_dense_table_create(opt.handle, int(shard_num), int(self_shard_id), C.byref(h)))
    return h.value


def save_sparse_table(table_handle, filepath, mode="txt"):
    """tn.core.save_sparse_table (core/main/py_wrapper.cc:211-215): the table in the reference's
    checkpoint format under <filepath>/sparse_table/<name or handle>/rank_0/."""
    _lib.check(_lib.load().tn_sparse_table_save(table_handle, str(filepath).encode(), str(mode).encode()))


def load_sparse_table(table_handle, filepath, mode="txt"):
    """tn.core.load_sparse_table (core/main/py_wrapper.cc:216-220)."""
    _lib.check(_lib.load().tn_sparse_table_load(table_handle, str(filepath).encode(), str(mode).encode()))


def save_dense_table(table_handle, filepath):
    """tn.core.save_dense_table (core/main/py_wrapper.cc:221-225): the dense table as the
    reference's text file <filepath>/dense_table/<handle>/0."""
    _lib.check(_lib.load().tn_dense_table_save(table_handle, str(filepath).encode()))


def load_dense_table(table_handle, filepath):
    """tn.core.load_dense_table (core/main/py_wrapper.cc:226-230)."""
    _lib.check(_lib.load().tn_dense_table_load(table_handle, str(filepath).encode()))


def show_decay(table_handle, delta_days):
    """tn.core.show_decay (core/main/py_wrapper.cc:259-262): every resident row of the sparse
    table ages by delta_days (SparseTable::ShowDecay)."""
    import torch

    _lib.check(_lib.load().tn_sparse_table_show_decay(
        table_handle, int(delta_days), C.c_void_p(torch.cuda.current_stream().cuda_stream)))


def reserve_sparse_table(table_handle, max_keys):
    """Sizes the HBM hash table for max_keys resident signs (no counterpart in
    the reference, whose host hash maps grow by themselves)."""
    _lib.check(_lib.load().tn_sparse_table_reserve(table_handle, int(max_keys)))


def clear_sparse_table(table_handle):
    """Drops every row of the table and frees its device memory (no counterpart in the
    reference, whose tables live in host memory until the process ends)."""
    _lib.check(_lib.load().tn_sparse_table_clear(table_handle))


def set_sparse_table_seed(table_handle, seed):
    _lib.check(_lib.load().tn_sparse_table_set_seed(table_handle, int(seed) & 0xFFFFFFFFFFFFFFFF))


def set_sparse_table_async(table_handle, async_pull):
    """With async_pull the pull op only enqueues its work (its counts and errors are collected by the next
    call on the table, or by sparse_table_sync); by default it waits for them, as the reference's op does."""
    _lib.check(_lib.load().tn_sparse_table_set_async(table_handle, 1 if async_pull else 0))


def set_sparse_table_small_batch_path(table_handle, enable):
    """Whether small batches take the path of few launches (the default) or the one every other batch takes:
    same results, a switch for measurements and tests."""
    _lib.check(_lib.load().tn_sparse_table_set_small_batch_path(table_handle, 1 if enable else 0))


def set_sparse_table_detached_updates(table_handle, enable):
    """With detached updates the update kernels of a large push run on the table's own streams, beside whatever
    the caller queues next (the analysis of the next pull's batch); the gradient tensors of the push must then
    stay untouched until the table's next pull, sync or other waiting call has returned.  Off by default."""
    _lib.check(_lib.load().tn_sparse_table_set_detached_updates(table_handle, 1 if enable else 0))


def set_sparse_table_exact_verify(table_handle, enable):
    """With exact verify a large pull keeps a copy of its signs and the push that follows compares the signs
    themselves instead of their fingerprints (16 bytes per 64 lookups).  Off by default."""
    _lib.check(_lib.load().tn_sparse_table_set_exact_verify(table_handle, 1 if enable else 0))


def sparse_table_key_count(table_handle):
    n = C.c_uint64()
    _lib.check(_lib.load().tn_sparse_table_key_count(table_handle, C.byref(n)))
    return n.value


def sparse_table_capacity(table_handle):
    n = C.c_uint64()
    _lib.check(_lib.load().tn_sparse_table_capacity(table_handle, C.byref(n)))
    return n.value


def sparse_table_row_layout(table_handle):
    w = C.c_int()
    s = C.c_int()
    _lib.check(_lib.load().tn_sparse_table_row_layout(table_handle, C.byref(w), C.byref(s)))
    return w.value, s.value
