"""ctypes binding of libtensornet_amd.so (the C ABI of include/tensornet_amd.h).

The library is loaded from the package directory, where `python -m
tensornet_amd.build` puts it.  There is no fallback: if the HIP library is
missing or fails to load, every operator of this package raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtensornet_amd.so")

TN_OK = 0
ERR_NAMES = {
    1: "TN_ERR_INVALID_ARGUMENT",
    2: "TN_ERR_BAD_HANDLE",
    3: "TN_ERR_DIM_MISMATCH",
    4: "TN_ERR_VAR_CAPACITY",
    5: "TN_ERR_UNKNOWN_KEY",
    6: "TN_ERR_TABLE_FULL",
    7: "TN_ERR_HIP",
    8: "TN_ERR_ALREADY_INIT",
    9: "TN_ERR_NOT_INIT",
    10: "TN_ERR_OUT_OF_MEMORY",
    11: "TN_ERR_UNSUPPORTED",
}


class TensorNetError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, code, message):
        super().__init__("%s (%d): %s" % (ERR_NAMES.get(code, "TN_ERR"), code, message))
        self.code = code
        self.message = message


class AdaGradParams(C.Structure):
    _fields_ = [
        ("learning_rate", C.c_float),
        ("show_decay_rate", C.c_float),
        ("show_threshold", C.c_float),
        ("initial_g2sum", C.c_float),
        ("initial_scale", C.c_float),
        ("epsilon", C.c_float),
        ("grad_decay_rate", C.c_float),
        ("mom_decay_rate", C.c_float),
        ("no_show_days", C.c_int32),
        ("elimination_logic", C.c_int32),
    ]


class AdamParams(C.Structure):
    _fields_ = [
        ("learning_rate", C.c_float),
        ("show_decay_rate", C.c_float),
        ("beta1", C.c_float),
        ("beta2", C.c_float),
        ("epsilon", C.c_float),
        ("initial_scale", C.c_float),
    ]


class FtrlParams(C.Structure):
    _fields_ = [
        ("learning_rate", C.c_float),
        ("show_decay_rate", C.c_float),
        ("show_threshold", C.c_float),
        ("beta", C.c_float),
        ("lambda1", C.c_float),
        ("lambda2", C.c_float),
        ("initial_scale", C.c_float),
    ]


class SignInfo(C.Structure):
    _fields_ = [("sign", C.c_uint64), ("batch_show", C.c_int32), ("batch_click", C.c_int32)]


_P = C.c_void_p
_PP = C.POINTER(C.c_void_p)
_I64P = C.POINTER(C.c_int64)

# name -> (restype, argtypes); every symbol include/tensornet_amd.h declares
SIGNATURES = {
    "tn_last_error": (C.c_char_p, []),
    "tn_version": (C.c_char_p, []),
    "tn_adagrad_params_default": (None, [C.POINTER(AdaGradParams)]),
    "tn_adam_params_default": (None, [C.POINTER(AdamParams)]),
    "tn_ftrl_params_default": (None, [C.POINTER(FtrlParams)]),
    "tn_opt_create_adagrad": (C.c_int, [C.POINTER(AdaGradParams), C.POINTER(C.c_int32)]),
    "tn_opt_create_adam": (C.c_int, [C.POINTER(AdamParams), C.POINTER(C.c_int32)]),
    "tn_opt_create_ftrl": (C.c_int, [C.POINTER(FtrlParams), C.POINTER(C.c_int32)]),
    "tn_opt_set_sparse_zero_init": (C.c_int, [C.c_int32, C.c_int]),
    "tn_opt_set_learning_rate": (C.c_int, [C.c_int32, C.c_float]),
    "tn_opt_get_learning_rate": (C.c_int, [C.c_int32, C.POINTER(C.c_float)]),
    "tn_sparse_table_create": (
        C.c_int,
        [C.c_int32, C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_char_p, C.POINTER(C.c_uint32)],
    ),
    "tn_sparse_table_reserve": (C.c_int, [C.c_uint32, C.c_uint64]),
    "tn_sparse_table_clear": (C.c_int, [C.c_uint32]),
    "tn_sparse_table_set_seed": (C.c_int, [C.c_uint32, C.c_uint64]),
    "tn_sparse_table_key_count": (C.c_int, [C.c_uint32, C.POINTER(C.c_uint64)]),
    "tn_sparse_table_capacity": (C.c_int, [C.c_uint32, C.POINTER(C.c_uint64)]),
    "tn_sparse_table_row_layout": (C.c_int, [C.c_uint32, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "tn_sparse_table_pull": (C.c_int, [C.c_uint32, _P, C.c_int64, C.c_int, _P, _P]),
    "tn_sparse_table_pull_static": (C.c_int, [C.c_uint32, _P, C.c_int64, C.c_int, _P, _P]),
    "tn_sparse_table_push": (C.c_int, [C.c_uint32, _P, _P, C.c_int64, C.c_int, _P]),
    "tn_sparse_table_load_rows": (C.c_int, [C.c_uint32, _P, _P, _P, C.c_int64, _P]),
    "tn_sparse_table_export_rows": (C.c_int, [C.c_uint32, _P, C.c_int64, _P, _P, _P, _P]),
    "tn_sparse_table_pull_op": (C.c_int, [C.c_uint32, C.c_int, _PP, _I64P, _PP, _I64P, C.c_int, _PP, _P]),
    "tn_sparse_table_push_op": (C.c_int, [C.c_uint32, C.c_int, _PP, _I64P, _PP, _I64P, C.c_int, _PP, _P]),
    "tn_sparse_table_combine_op": (C.c_int, [C.c_uint32, C.c_int, _PP, _I64P, _PP, _PP, _I64P, C.c_int, C.c_int64,
                                             C.c_int, _PP, _P]),
    "tn_sparse_table_push_pooled_op": (C.c_int, [C.c_uint32, C.c_int, _PP, _I64P, _PP, _PP, C.c_int64, C.c_int,
                                                 C.c_int, _PP, _P]),
    "tn_sparse_table_show_decay": (C.c_int, [C.c_uint32, C.c_int, _P]),
    "tn_sparse_table_delete_by_show": (C.c_int, [C.c_uint32, _P, C.c_int64, _P, _P]),
    "tn_sparse_table_save": (C.c_int, [C.c_uint32, C.c_char_p, C.c_char_p]),
    "tn_sparse_table_load": (C.c_int, [C.c_uint32, C.c_char_p, C.c_char_p]),
    "tn_sparse_table_export_range": (C.c_int, [C.c_uint32, C.c_uint64, C.c_uint64, C.c_int, _P, _P, _P,
                                               C.POINTER(C.c_uint64), _P]),
    "tn_sparse_table_name": (C.c_int, [C.c_uint32, C.c_char_p, C.c_int]),
    "tn_sparse_table_optimizer": (C.c_int, [C.c_uint32, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "tn_sparse_table_sync": (C.c_int, [C.c_uint32]),
    "tn_sparse_table_last_unique_counts": (C.c_int, [C.c_uint32, C.c_int, _I64P]),
    "tn_sparse_table_set_async": (C.c_int, [C.c_uint32, C.c_int]),
    "tn_sparse_table_set_small_batch_path": (C.c_int, [C.c_uint32, C.c_int]),
    "tn_sparse_table_set_detached_updates": (C.c_int, [C.c_uint32, C.c_int]),
    "tn_sparse_table_set_exact_verify": (C.c_int, [C.c_uint32, C.c_int]),
    "tn_dense_table_create": (C.c_int, [C.c_int32, C.c_int, C.c_int, C.POINTER(C.c_uint32)]),
    "tn_dense_table_init": (C.c_int, [C.c_uint32, C.c_int, _PP, _I64P, _P]),
    "tn_dense_table_push_pull": (C.c_int, [C.c_uint32, C.c_int, _PP, _PP, _I64P, C.c_float, _P]),
    "tn_dense_table_total_elements": (C.c_int, [C.c_uint32, _I64P]),
    "tn_dense_table_range": (C.c_int, [C.c_uint32, _I64P, _I64P]),
    "tn_dense_table_get_weight": (C.c_int, [C.c_uint32, _P, _P]),
    "tn_dense_table_set_weight": (C.c_int, [C.c_uint32, _P, _P]),
    "tn_dense_table_get_state": (C.c_int, [C.c_uint32, _P, _P, _P, _P]),
    "tn_dense_table_save": (C.c_int, [C.c_uint32, C.c_char_p]),
    "tn_dense_table_load": (C.c_int, [C.c_uint32, C.c_char_p]),
    "tn_profile_enable": (C.c_int, [C.c_int]),
    "tn_profile_reset": (C.c_int, []),
    "tn_profile_summary": (C.c_int, [C.c_char_p, C.c_size_t]),
}

_lib = None


def load():
    """Returns the loaded library; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "tensornet_amd: %s not found -- build it with `python -m tensornet_amd.build` "
            "(there is no CPU fallback)" % LIB_PATH
        )
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc):
    if rc != TN_OK:
        raise TensorNetError(rc, load().tn_last_error().decode("utf-8", "replace"))


def ptr_array(ptrs):
    arr = (C.c_void_p * len(ptrs))()
    for i, p in enumerate(ptrs):
        arr[i] = p
    return arr


def i64_array(vals):
    arr = (C.c_int64 * len(vals))()
    for i, v in enumerate(vals):
        arr[i] = int(v)
    return arr


def profile_summary():
    """{kernel name: (launches, total milliseconds)} of the launches recorded since the last reset."""
    buf = C.create_string_buffer(1 << 16)
    check(load().tn_profile_summary(buf, len(buf)))
    out = {}
    for line in buf.value.decode().splitlines():
        name, count, ms = line.split("\t")
        out[name.strip("()")] = (int(count), float(ms))
    return out
