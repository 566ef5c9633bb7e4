"""hpcdnn for AMD MI355X: FP32 SGEMM, ABFT-SGEMM, SAXPY and SDOT as hand-written gfx950 HIP kernels.

``blas`` mirrors the reference's kernel entry points on torch device tensors;
``_lib`` is the raw ctypes binding of the C ABI (``include/hpcdnn.h``).
"""
from . import _lib  # noqa: F401
from ._lib import HpcdnnError, build  # noqa: F401

__all__ = ["blas", "HpcdnnError", "build"]


def __getattr__(name):
    if name == "blas":  # torch is imported only when the tensor-level API is used
        import importlib

        return importlib.import_module(".blas", __name__)
    raise AttributeError(name)
