"""MI355X-native MergePath-SpMM: Python face of libmpspmm.so.

The directory name carries a hyphen, so the package is imported under the
name ``mergepath_spmm_amd`` through ``__graft_entry__.load_package()``.
"""
from . import _cabi, build, graphs  # noqa: F401
from ._cabi import MpsError  # noqa: F401

__all__ = ["_cabi", "build", "graphs", "MpsError"]


def __getattr__(name):
    # spmm needs torch; load it on first use so that host-only users skip the import
    if name == "spmm":
        import importlib
        return importlib.import_module(__name__ + ".spmm")
    raise AttributeError(name)
