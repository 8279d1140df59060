"""tensornet_amd: TensorNet's sparse pull / push and dense update path on MI355X.

`core` mirrors the reference's `tn.core` configuration functions, `ops` its
four TensorFlow ops.  Both call the HIP library through the C ABI declared in
include/tensornet_amd.h; there is no CPU fallback.
"""
from . import core  # noqa: F401
from ._lib import TensorNetError, load  # noqa: F401

__all__ = ["core", "ops", "TensorNetError", "load"]


def __getattr__(name):
    if name == "ops":  # imports torch; keep `import tensornet_amd` light
        import importlib

        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
