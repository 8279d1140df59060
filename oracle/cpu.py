"""ctypes front end of oracle/liboracle.so (see oracle/oracle.cc).

TEST INFRASTRUCTURE: the checker the HIP path is compared with, and the timed
CPU baseline of bench.py.  Works on numpy arrays.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
# the same source built with the reference's Release flags: what bench.py times as the CPU baseline
TIMED_LIB_PATH = os.path.join(_HERE, "liboracle_timed.so")
TIMED_FLAGS = "g++ -O3 -DNDEBUG -march=x86-64-v2 -mavx -std=c++14 (CMakeLists.txt:224-238 of the reference)"

ADAGRAD, ADAM, FTRL = 0, 1, 2

sign_info_dtype = np.dtype([("sign", "<u8"), ("batch_show", "<i4"), ("batch_click", "<i4")])

_lib = None
_timed = False


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def load(timed=False):
    """The checker's library; timed=True switches every later call of this module to the build with the
    reference's Release flags (bench.py's CPU baseline; parity tests keep the default build)."""
    global _lib, _timed
    if _lib is not None and (not timed or _timed):
        return _lib
    path = TIMED_LIB_PATH if timed else LIB_PATH
    if not os.path.exists(path):
        build()
    lib = C.CDLL(path)
    _timed = bool(timed)
    P = C.c_void_p
    lib.orc_table_create.restype = P
    lib.orc_table_create.argtypes = [C.c_int, P, C.c_int, C.c_int, C.c_int, C.c_uint64, C.c_uint64]
    lib.orc_table_destroy.argtypes = [P]
    lib.orc_table_weight_floats.argtypes = [P]
    lib.orc_table_state_floats.argtypes = [P]
    lib.orc_table_key_count.restype = C.c_uint64
    lib.orc_table_key_count.argtypes = [P]
    lib.orc_table_serialize_block.restype = C.c_int64
    lib.orc_table_serialize_block.argtypes = [P, C.c_int, C.c_int, P, C.c_int64]
    lib.orc_table_deserialize_block.restype = C.c_int64
    lib.orc_table_deserialize_block.argtypes = [P, C.c_int, P, C.c_int64]
    lib.orc_table_show_decay.restype = None
    lib.orc_table_show_decay.argtypes = [P, C.c_int]
    lib.orc_table_delete_by_show.restype = None
    lib.orc_table_delete_by_show.argtypes = [P, P, C.c_int64, P]
    lib.orc_table_set_rows.argtypes = [P, P, P, P, C.c_int64]
    lib.orc_table_get_rows.argtypes = [P, P, C.c_int64, P, P, P]
    lib.orc_table_pull.argtypes = [P, P, C.c_int64, C.c_int, P]
    lib.orc_table_push.argtypes = [P, P, P, C.c_int64, C.c_int]
    lib.orc_pull_remap.restype = C.c_int64
    lib.orc_pull_remap.argtypes = [P, C.c_int64, P, P]
    lib.orc_push_remap.restype = C.c_int64
    lib.orc_push_remap.argtypes = [P, P, C.c_int64, P]
    lib.orc_pull_op.argtypes = [P, C.c_int, P, P, P, P, C.c_int, P, P]
    lib.orc_push_op.argtypes = [P, C.c_int, P, P, P, C.c_int, P, P]
    lib.orc_dense_create.restype = P
    lib.orc_dense_create.argtypes = [C.c_int, P, C.c_int64]
    lib.orc_dense_destroy.argtypes = [P]
    lib.orc_dense_set_weight.argtypes = [P, P]
    lib.orc_dense_get_weight.argtypes = [P, P]
    lib.orc_dense_apply.argtypes = [P, P, C.c_float]
    lib.orc_dense_num_blocks.argtypes = [P]
    lib.orc_dense_get_state.argtypes = [P, C.c_int, P]
    lib.orc_dense_serialize.restype = C.c_int64
    lib.orc_dense_serialize.argtypes = [P, C.c_int, C.c_int, P, C.c_int64]
    lib.orc_dense_deserialize.argtypes = [P, C.c_int, C.c_int, P, C.c_int64]
    lib.orc_dense_get_powers.argtypes = [P, C.c_int, P]
    _lib = lib
    return lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _ptrs(arrays):
    arr = (C.c_void_p * len(arrays))()
    for i, a in enumerate(arrays):
        arr[i] = a.ctypes.data
    return arr


def _params(kind, **kw):
    """Packs hyper-parameters in the order oracle.cc's FillOpt reads them."""
    if kind == ADAGRAD:
        vals = [
            kw.get("learning_rate", 0.01),
            kw.get("initial_g2sum", 0.0),
            kw.get("initial_scale", 1.0),
            kw.get("epsilon", 1e-8),
            kw.get("grad_decay_rate", 1.0),
            kw.get("mom_decay_rate", 1.0),
        ]
    elif kind == ADAM:
        vals = [
            kw.get("learning_rate", 0.01),
            kw.get("beta1", 0.9),
            kw.get("beta2", 0.999),
            kw.get("epsilon", 1e-8),
            kw.get("initial_scale", 1.0),
        ]
    else:
        vals = [
            kw.get("learning_rate", 0.01),
            kw.get("beta", 1.0),
            kw.get("lambda1", 0.1),
            kw.get("lambda2", 1.0),
            kw.get("initial_scale", 1.0),
        ]
    tail = [
        kw.get("show_decay_rate", 0.98),
        kw.get("show_threshold", 0.0),
        float(kw.get("no_show_days", 1000)),
        float(kw.get("elimination_logic", 0)),
    ]
    return np.asarray(vals + [0.0] * (8 - len(vals)) + tail, dtype=np.float32)


def pull_remap(values):
    """SparsePullVarInfo: (mapped ids int64[L], distinct signs uint64[U])."""
    values = np.ascontiguousarray(values, dtype=np.int64)
    mapped = np.empty_like(values)
    signs = np.empty(values.shape[0], dtype=np.uint64)
    u = load().orc_pull_remap(_p(values), values.shape[0], _p(mapped), _p(signs))
    return mapped, signs[:u].copy()


def push_remap(values, labels):
    """SparsePushVarInfo: structured array (sign, batch_show, batch_click)[U]."""
    values = np.ascontiguousarray(values, dtype=np.int64)
    labels = np.ascontiguousarray(labels, dtype=np.int64)
    infos = np.empty(values.shape[0], dtype=sign_info_dtype)
    u = load().orc_push_remap(_p(values), _p(labels), values.shape[0], _p(infos))
    return infos[:u].copy()


class Table(object):
    """One SparseTable of the reference with its 8-block optimizer kernel."""

    def __init__(self, kind, dim, use_cvm=False, zero_init=False, seed=1, buckets=15485863, **hyper):
        self.kind = kind
        self.dim = dim
        self._params = _params(kind, **hyper)
        self._h = load().orc_table_create(
            kind, _p(self._params), dim, int(use_cvm), int(zero_init), seed, buckets
        )
        self.wf = load().orc_table_weight_floats(self._h)
        self.sf = load().orc_table_state_floats(self._h)

    def __del__(self):
        # (at interpreter exit the module's globals may be gone before the last table is)
        if getattr(self, "_h", None) and load is not None:
            load().orc_table_destroy(self._h)
            self._h = None

    def key_count(self):
        return int(load().orc_table_key_count(self._h))

    def serialize_block(self, block, mode="txt"):
        """Uncompressed checkpoint stream of hash block 0..7, as bytes."""
        lib = load()
        n = lib.orc_table_serialize_block(self._h, block, int(mode == "bin"), None, 0)
        buf = np.zeros(max(1, n), dtype=np.uint8)
        lib.orc_table_serialize_block(self._h, block, int(mode == "bin"), _p(buf), n)
        return buf[:n].tobytes()

    def deserialize_block(self, data, mode="txt"):
        buf = np.frombuffer(data, dtype=np.uint8)
        n = load().orc_table_deserialize_block(self._h, int(mode == "bin"), _p(np.ascontiguousarray(buf)), len(buf))
        if n < 0:
            raise ValueError("checkpoint stream was written with another optimizer or dim")
        return int(n)

    def save(self, filepath, ident, mode="txt"):
        """SparseTable::Save (core/ps/table/sparse_table.cc:84-108): eight gzip files
        <filepath>/sparse_table/<ident>/rank_0/block_<i>.gz."""
        import gzip

        d = os.path.join(filepath, "sparse_table", str(ident), "rank_0")
        os.makedirs(d, exist_ok=True)
        for b in range(8):
            with gzip.open(os.path.join(d, "block_%d.gz" % b), "wb") as f:
                f.write(self.serialize_block(b, mode))

    def load(self, filepath, ident, mode="txt", prefix="block_", suffix=""):
        """SparseTable::Load (sparse_table.cc:110-137); the caller names prefix / suffix / mode,
        which the reference derives from the first file name (optimizer_kernel.h:496-520)."""
        import gzip

        d = os.path.join(filepath, "sparse_table", str(ident), "rank_0")
        n = 0
        for b in range(8):
            with gzip.open(os.path.join(d, "%s%d%s.gz" % (prefix, b, suffix)), "rb") as f:
                n += self.deserialize_block(f.read(), mode)
        return n

    def show_decay(self, delta_days):
        load().orc_table_show_decay(self._h, int(delta_days))

    def delete_by_show(self, signs):
        signs = np.ascontiguousarray(signs, dtype=np.uint64)
        out = np.zeros(len(signs), dtype=np.uint8)
        load().orc_table_delete_by_show(self._h, _p(signs), len(signs), _p(out))
        return out.astype(bool)

    def set_rows(self, signs, w, state=None):
        signs = np.ascontiguousarray(signs, dtype=np.uint64)
        w = np.ascontiguousarray(w, dtype=np.float32).reshape(len(signs), self.wf)
        if state is not None:
            state = np.ascontiguousarray(state, dtype=np.float32).reshape(len(signs), self.sf)
        load().orc_table_set_rows(self._h, _p(signs), _p(w), _p(state), len(signs))

    def get_rows(self, signs):
        signs = np.ascontiguousarray(signs, dtype=np.uint64)
        w = np.zeros((len(signs), self.wf), dtype=np.float32)
        st = np.zeros((len(signs), self.sf), dtype=np.float32)
        found = np.zeros(len(signs), dtype=np.uint8)
        load().orc_table_get_rows(self._h, _p(signs), len(signs), _p(w), _p(st), _p(found))
        return w, st, found

    def pull(self, signs, dim=None):
        signs = np.ascontiguousarray(signs, dtype=np.uint64)
        dim = self.wf if dim is None else dim
        out = np.empty((len(signs), dim), dtype=np.float32)
        load().orc_table_pull(self._h, _p(signs), len(signs), dim, _p(out))
        return out

    def push(self, infos, grads):
        infos = np.ascontiguousarray(infos, dtype=sign_info_dtype)
        grads = np.ascontiguousarray(grads, dtype=np.float32)
        return load().orc_table_push(self._h, _p(infos), _p(grads), len(infos), grads.shape[1])

    def pull_op(self, values, vars):
        """values: list of int64 arrays; vars: list of float32 [rows, dim] arrays (written
        in place).  Returns (status, mapped list, distinct counts)."""
        n = len(values)
        values = [np.ascontiguousarray(v, dtype=np.int64) for v in values]
        mapped = [np.empty_like(v) for v in values]
        lens = np.asarray([len(v) for v in values], dtype=np.int64)
        rows = np.asarray([v.shape[0] for v in vars], dtype=np.int64)
        counts = np.zeros(n, dtype=np.int64)
        rc = load().orc_pull_op(
            self._h, n, _ptrs(values), _p(lens), _ptrs(vars), _p(rows), vars[0].shape[1], _ptrs(mapped), _p(counts)
        )
        return rc, mapped, counts

    def push_op(self, values, grads, labels):
        n = len(values)
        values = [np.ascontiguousarray(v, dtype=np.int64) for v in values]
        labels = [np.ascontiguousarray(l, dtype=np.int64) for l in labels]
        grads = [np.ascontiguousarray(g, dtype=np.float32) for g in grads]
        lens = np.asarray([len(v) for v in values], dtype=np.int64)
        counts = np.zeros(n, dtype=np.int64)
        rc = load().orc_push_op(
            self._h, n, _ptrs(values), _p(lens), _ptrs(grads), grads[0].shape[1], _ptrs(labels), _p(counts)
        )
        return rc, counts


class Dense(object):
    """DenseTable of one worker: 8 optimizer blocks over a flat array."""

    def __init__(self, kind, total, **hyper):
        self.total = total
        self._params = _params(kind, **hyper)
        self._h = load().orc_dense_create(kind, _p(self._params), total)

    def __del__(self):
        if getattr(self, "_h", None):
            load().orc_dense_destroy(self._h)
            self._h = None

    def num_blocks(self):
        return load().orc_dense_num_blocks(self._h)

    def set_weight(self, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        assert w.size == self.total
        load().orc_dense_set_weight(self._h, _p(w))

    def get_weight(self):
        w = np.empty(self.total, dtype=np.float32)
        load().orc_dense_get_weight(self._h, _p(w))
        return w

    def apply(self, grad, lr):
        grad = np.ascontiguousarray(grad, dtype=np.float32)
        assert grad.size == self.total
        load().orc_dense_apply(self._h, _p(grad), lr)

    def get_state(self, which):
        out = np.zeros(self.total, dtype=np.float32)
        load().orc_dense_get_state(self._h, which, _p(out))
        return out

    def beta_powers(self, block=0):
        out = np.zeros(2, dtype=np.float32)
        load().orc_dense_get_powers(self._h, block, _p(out))
        return float(out[0]), float(out[1])

    def serialize(self, rank_num=1, table_total=None):
        """Text of the checkpoint file DenseTable::Save writes (core/ps/table/dense_table.cc:103-128).
        With several shards this object is one shard's kernel (its range of the table) and
        table_total the size of the whole table."""
        lib = load()
        tt = self.total if table_total is None else int(table_total)
        n = lib.orc_dense_serialize(self._h, rank_num, tt, None, 0)
        buf = np.zeros(max(1, n), dtype=np.uint8)
        lib.orc_dense_serialize(self._h, rank_num, tt, _p(buf), n)
        return buf[:n].tobytes()

    def deserialize(self, data, shard_num=1, table_total=None):
        """DenseTable::Load (dense_table.cc:130-157) into a table of the file's total."""
        buf = np.ascontiguousarray(np.frombuffer(data, dtype=np.uint8))
        tt = self.total if table_total is None else int(table_total)
        rc = load().orc_dense_deserialize(self._h, shard_num, tt, _p(buf), len(buf))
        if rc != 0:
            raise ValueError({-1: "total elements", -2: "shard count", -3: "optimizer", -4: "block length"}[rc]
                             + " of the checkpoint differs from the table's")

    def save(self, filepath, handle, shard=0):
        d = os.path.join(filepath, "dense_table", str(handle))
        os.makedirs(d, exist_ok=True)
        with open(os.path.join(d, str(shard)), "wb") as f:
            f.write(self.serialize())

    def load(self, filepath, handle, shard=0):
        with open(os.path.join(filepath, "dense_table", str(handle), str(shard)), "rb") as f:
            self.deserialize(f.read())
