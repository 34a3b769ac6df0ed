"""Host-side graph inputs: .csr text files, seeded synthetic graphs, fills.

Thin wrappers over the host half of the C ABI; arrays come back as numpy.
"""
import ctypes

import numpy as np

from . import _cabi
from ._cabi import check

# The five benchmark graphs, as generator specs.
CONFIG_SPECS = {
    "er_4096": "er:n=4096,deg=8",
    "chunglu_233k": "chunglu:n=232965,nnz=114600000,gamma=2.1,dmax=20000",
    "blockdiag_1178": "blockdiag:blocks=1178,min=100,max=600,deg=5",
    "rmat_s20": "rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19",
    "rmat_s22": "rmat:scale=22,ef=16,a=0.57,b=0.19,c=0.19",
}


def _take(handle):
    L = _cabi.lib()
    n, nnz, md = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    check(L.mps_graph_dims(handle, ctypes.byref(n), ctypes.byref(nnz), ctypes.byref(md)), "mps_graph_dims")
    rp = np.ctypeslib.as_array(ctypes.cast(L.mps_graph_row_ptr(handle), _cabi.c_int_p), (n.value + 1,)).copy()
    if nnz.value:
        ci = np.ctypeslib.as_array(ctypes.cast(L.mps_graph_col_idx(handle), _cabi.c_int_p), (nnz.value,)).copy()
    else:
        ci = np.zeros(0, dtype=np.int32)
    L.mps_graph_free(handle)
    return rp, ci, md.value


def generate(spec, seed=1):
    """(row_ptr, col_idx, max_degree) of the graph a spec string and a seed name."""
    h = ctypes.c_void_p()
    check(_cabi.lib().mps_graph_generate(spec.encode(), ctypes.c_uint64(seed), ctypes.byref(h)),
          "mps_graph_generate(%s)" % spec)
    return _take(h)


def from_edges(src, dst):
    """Edge list -> (row_ptr, col_idx, max_degree): rows sorted, repeated edges
    merged, square (what scripts/npz_to_csr.py:14-20 gets from scipy)."""
    s = np.ascontiguousarray(src, dtype=np.int64)
    d = np.ascontiguousarray(dst, dtype=np.int64)
    if s.size != d.size:
        raise ValueError("src and dst differ in length")
    h = ctypes.c_void_p()
    check(_cabi.lib().mps_graph_from_edges(s.ctypes.data, d.ctypes.data, ctypes.c_int64(s.size), ctypes.byref(h)),
          "mps_graph_from_edges")
    return _take(h)


def read_csr(path):
    """Two-line .csr text -> (row_ptr, col_idx, max_degree)."""
    h = ctypes.c_void_p()
    check(_cabi.lib().mps_graph_from_csr_file(str(path).encode(), ctypes.byref(h)),
          "mps_graph_from_csr_file(%s)" % path)
    return _take(h)


def read_csr_header(path):
    n, nnz = ctypes.c_int(), ctypes.c_int()
    check(_cabi.lib().mps_csr_read_header(str(path).encode(), ctypes.byref(n), ctypes.byref(nnz)),
          "mps_csr_read_header(%s)" % path)
    return n.value, nnz.value


def write_csr(path, row_ptr, col_idx):
    rp = np.ascontiguousarray(row_ptr, dtype=np.int32)
    ci = np.ascontiguousarray(col_idx, dtype=np.int32)
    check(_cabi.lib().mps_csr_write(str(path).encode(), int(rp.size - 1), rp.ctypes.data, ci.ctypes.data),
          "mps_csr_write(%s)" % path)


def fill_uniform_f32(n, seed, lo, hi):
    out = np.empty(int(n), dtype=np.float32)
    check(_cabi.lib().mps_fill_uniform_f32(out.ctypes.data, out.size, ctypes.c_uint64(seed), lo, hi),
          "mps_fill_uniform_f32")
    return out


def fill_uniform_f16(n, seed, lo, hi):
    out = np.empty(int(n), dtype=np.float16)
    check(_cabi.lib().mps_fill_uniform_f16(out.ctypes.data, out.size, ctypes.c_uint64(seed), lo, hi),
          "mps_fill_uniform_f16")
    return out


def num_partitions(n_rows, nnz, cost):
    """cost -> P (src/MergePathSpMM.cu:138-139)."""
    p = ctypes.c_int()
    check(_cabi.lib().mps_num_partitions(int(n_rows), int(nnz), int(cost), ctypes.byref(p)), "mps_num_partitions")
    return p.value


def items_per_partition(n_rows, nnz, P):
    v = ctypes.c_int()
    check(_cabi.lib().mps_items_per_partition(int(n_rows), int(nnz), int(P), ctypes.byref(v)),
          "mps_items_per_partition")
    return v.value


def max_threads_per_wave(K, elem_bytes=4):
    v = ctypes.c_int()
    check(_cabi.lib().mps_max_threads_per_wave(int(K), int(elem_bytes), ctypes.byref(v)),
          "mps_max_threads_per_wave")
    return v.value


def rowwise_bounds(n_rows, num_waves):
    s = np.empty(num_waves, dtype=np.int32)
    e = np.empty(num_waves, dtype=np.int32)
    check(_cabi.lib().mps_rowwise_bounds(int(n_rows), int(num_waves), s.ctypes.data, e.ctypes.data),
          "mps_rowwise_bounds")
    return s, e
