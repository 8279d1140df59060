"""The C-ABI library loads without a GPU and exports every entry point that
include/tensornet_amd.h declares; host-only entry points behave."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tensornet_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import tensornet_amd
    from tensornet_amd import _lib

    lib = tensornet_amd.load()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_lib.SIGNATURES) == names


def test_optimizer_factories_and_defaults():
    import tensornet_amd as tn
    from tensornet_amd import _lib

    lib = tn.load()
    p = _lib.AdaGradParams()
    lib.tn_adagrad_params_default(C.byref(p))
    # core/main/py_wrapper.cc:94-104
    assert (round(p.learning_rate, 6), round(p.show_decay_rate, 6), p.initial_g2sum, p.initial_scale) == (0.01, 0.98, 0.0, 1.0)
    assert (p.no_show_days, p.elimination_logic, p.grad_decay_rate, p.mom_decay_rate) == (1000, 0, 1.0, 1.0)
    a = _lib.AdamParams()
    lib.tn_adam_params_default(C.byref(a))
    assert (round(a.beta1, 6), round(a.beta2, 6), round(a.epsilon, 12)) == (0.9, 0.999, 1e-8)
    f = _lib.FtrlParams()
    lib.tn_ftrl_params_default(C.byref(f))
    assert (f.beta, round(f.lambda1, 6), f.lambda2, f.initial_scale) == (1.0, 0.1, 1.0, 1.0)

    opt = tn.core.AdaGrad(learning_rate=0.05, initial_g2sum=0.1, not_a_parameter=3)
    assert abs(tn.core.get_opt_learning_rate(opt) - 0.05) < 1e-9
    with pytest.raises(ValueError):
        tn.core.AdaGrad(elimination_logic=2)
    p.elimination_logic = 5
    h = C.c_int32()
    assert lib.tn_opt_create_adagrad(C.byref(p), C.byref(h)) == 1
    assert b"elimination_logic" in lib.tn_last_error()


def test_bad_handles_return_codes_not_aborts():
    import tensornet_amd as tn

    lib = tn.load()
    n = C.c_uint64()
    assert lib.tn_sparse_table_key_count(12345, C.byref(n)) == 2
    assert lib.tn_sparse_table_sync(12345) == 2
    h = C.c_uint32()
    assert lib.tn_sparse_table_create(999, b"x", 8, 0, 1, 0, b"", C.byref(h)) == 2
    assert lib.tn_dense_table_create(999, 1, 0, C.byref(h)) == 2
    with pytest.raises(tn.TensorNetError) as e:
        tn.core.create_sparse_table(tn.core.Adam(), "t", 0)
    assert e.value.code == 1


def test_embedding_group_shares_one_table():
    import tensornet_amd as tn

    opt = tn.core.AdaGrad()
    a = tn.core.create_sparse_table(opt, "a", 8, False, "grp-shared")
    b = tn.core.create_sparse_table(opt, "b", 8, False, "grp-shared")
    c = tn.core.create_sparse_table(opt, "c", 8, False, "")
    assert a == b and c != a  # sparse_table.cc:175-180
    assert tn.core.sparse_table_row_layout(a) == (8, 4)
    assert tn.core.sparse_table_row_layout(tn.core.create_sparse_table(tn.core.Adam(), "d", 16)) == (16, 34)
