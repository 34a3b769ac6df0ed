"""ctypes front end of the CPU oracle (oracle/mp_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark, never by the shipped package or drivers.
Each function cites the reference lines its C body follows.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmp_oracle.so")
_lib = None


def build(force=False):
    """Compile oracle/mp_oracle.c with gcc (make)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_half_to_double.restype = ctypes.c_double
        _lib.orc_half_to_double.argtypes = [ctypes.c_uint16]
    return _lib


def _ip(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def num_partitions(n_rows, nnz, cost):
    """src/MergePathSpMM.cu:138-139."""
    return int(lib().orc_num_partitions(int(n_rows), int(nnz), int(cost)))


def merge_path_search(diagonal, row_ptr, nnz):
    """src/MergePathSpMM.cu:280-297 (literal loop, NZ_INDICES materialised)."""
    rp = _i32(row_ptr)
    nz = np.arange(max(nnz, 1), dtype=np.int32)
    x = ctypes.c_int()
    y = ctypes.c_int()
    lib().orc_merge_path_search(int(diagonal), _ip(rp), _ip(nz), int(rp.size), int(nnz),
                                ctypes.byref(x), ctypes.byref(y))
    return x.value, y.value


def merge_path_closed_form(diagonal, row_ptr):
    rp = _i32(row_ptr)
    x = ctypes.c_int()
    y = ctypes.c_int()
    lib().orc_merge_path_closed_form(int(diagonal), _ip(rp), int(rp.size),
                                     ctypes.byref(x), ctypes.byref(y))
    return x.value, y.value


def merge_path_walk(row_ptr, nnz):
    rp = _i32(row_ptr)
    total = rp.size + nnz
    xs = np.empty(total + 1, dtype=np.int32)
    ys = np.empty(total + 1, dtype=np.int32)
    lib().orc_merge_path_walk(_ip(rp), int(rp.size), int(nnz), _ip(xs), _ip(ys))
    return xs, ys


def partition_coords(row_ptr, nnz, P):
    """Partition boundary coordinates, diagonals as in src/MergePathSpMM.cu:327-334."""
    rp = _i32(row_ptr)
    xs = np.empty(P + 1, dtype=np.int32)
    ys = np.empty(P + 1, dtype=np.int32)
    lib().orc_partition_coords(_ip(rp), int(rp.size - 1), int(nnz), int(P), _ip(xs), _ip(ys))
    return xs, ys


SCHED_FIELDS = ("feature_start", "feature_start_num", "feature_end", "feature_end_num",
                "start_row", "end_row")


def generate_mp_sched(row_ptr, nnz, P):
    """src/MergePathSpMM.cu:300-385; dict of the six int32[P] arrays."""
    rp = _i32(row_ptr)
    out = [np.zeros(P, dtype=np.int32) for _ in range(6)]
    lib().orc_generate_mp_sched(_ip(rp), int(rp.size - 1), int(nnz), int(P), *[_ip(a) for a in out])
    return dict(zip(SCHED_FIELDS, out))


def spmm_f64(row_ptr, col_idx, val, X, want_abs=False):
    """fp64 row loop, explicit values; returns Y (and the |.|-sum scale)."""
    rp, ci = _i32(row_ptr), _i32(col_idx)
    v = np.ascontiguousarray(val, dtype=np.float32)
    Xc = np.ascontiguousarray(X, dtype=np.float32)
    n, K = rp.size - 1, Xc.shape[1]
    Y = np.empty((n, K), dtype=np.float64)
    A = np.empty((n, K), dtype=np.float64) if want_abs else None
    lib().orc_spmm_f64(_ip(rp), _ip(ci), _ip(v), _ip(Xc), int(n), int(K), _ip(Y),
                       _ip(A) if want_abs else None)
    return (Y, A) if want_abs else Y


def spmm_f64_f16in(row_ptr, col_idx, val_h, X_h, want_abs=False):
    """fp64 row loop over half inputs (numpy float16 arrays)."""
    rp, ci = _i32(row_ptr), _i32(col_idx)
    v = np.ascontiguousarray(val_h, dtype=np.float16).view(np.uint16)
    Xc = np.ascontiguousarray(X_h, dtype=np.float16).view(np.uint16)
    n, K = rp.size - 1, Xc.shape[1]
    Y = np.empty((n, K), dtype=np.float64)
    A = np.empty((n, K), dtype=np.float64) if want_abs else None
    lib().orc_spmm_f64_f16in(_ip(rp), _ip(ci), _ip(v), _ip(Xc), int(n), int(K), _ip(Y),
                             _ip(A) if want_abs else None)
    return (Y, A) if want_abs else Y


def spmm_mergepath_f32(row_ptr, col_idx, val, X, P):
    """Reference kernel structure (src/MergePathSpMM.cu:426-477), explicit values."""
    rp, ci = _i32(row_ptr), _i32(col_idx)
    v = np.ascontiguousarray(val, dtype=np.float32)
    Xc = np.ascontiguousarray(X, dtype=np.float32)
    n, K = rp.size - 1, Xc.shape[1]
    Y = np.empty((n, K), dtype=np.float32)
    lib().orc_spmm_mergepath_f32(_ip(rp), _ip(ci), _ip(v), _ip(Xc), int(n), int(ci.size), int(K),
                                 int(P), _ip(Y))
    return Y


def spmm_f32_mt(row_ptr, col_idx, val, X, threads=0, out=None):
    """Multithreaded fp32 CSR x dense (the timed CPU baseline)."""
    rp, ci = _i32(row_ptr), _i32(col_idx)
    v = np.ascontiguousarray(val, dtype=np.float32)
    Xc = np.ascontiguousarray(X, dtype=np.float32)
    n, K = rp.size - 1, Xc.shape[1]
    Y = out if out is not None else np.empty((n, K), dtype=np.float32)
    if threads <= 0:
        threads = max_threads()
    lib().orc_spmm_f32_mt(_ip(rp), _ip(ci), _ip(v), _ip(Xc), int(n), int(K), _ip(Y), int(threads))
    return Y


def max_threads():
    return int(lib().orc_max_threads())


def rowwise_bounds(num_nodes, num_warps):
    """src/row_wise.cu:211-213."""
    s = np.empty(num_warps, dtype=np.int32)
    e = np.empty(num_warps, dtype=np.int32)
    lib().orc_rowwise_bounds(int(num_nodes), int(num_warps), _ip(s), _ip(e))
    return s, e


def calculate_part_num(part_size, row_ptr):
    """src/nz_splitting.cu:299-316."""
    rp = _i32(row_ptr)
    return int(lib().orc_calculate_part_num(int(part_size), _ip(rp), int(rp.size - 1)))


def build_part(part_size, row_ptr):
    """src/nz_splitting.cu:256-297 -> (partPtr[numParts+1], part2Node[numParts])."""
    rp = _i32(row_ptr)
    n = calculate_part_num(part_size, rp)
    pp = np.empty(n + 1, dtype=np.int32)
    pn = np.empty(max(n, 1), dtype=np.int32)
    lib().orc_build_part(int(part_size), _ip(rp), int(rp.size - 1), _ip(pp), _ip(pn))
    return pp, pn[:n]


def degree_values(row_ptr, col_idx, mode="product", dtype=np.float32):
    """The reference's implicit edge weight as an array.  degrees[i] =
    row_ptr[i+1] - row_ptr[i] (src/MergePathSpMM.cu:183-185); weight of
    nonzero (r, c) = float(deg r) * float(deg c), one rounded fp32 product
    (:450,459).  dtype=np.float16: both degrees converted to half and
    multiplied in half (src/MergePathSpMM_fp16.cu:451,460; infinity beyond
    65504).  mode="gcn": 1 / sqrt(deg r * deg c) in fp32, 0 where a degree
    is 0 (no reference counterpart)."""
    rp, ci = _i32(row_ptr), _i32(col_idx)
    deg = np.diff(rp)
    rows = np.repeat(np.arange(rp.size - 1), deg)
    with np.errstate(over="ignore", divide="ignore", invalid="ignore"):
        if mode == "gcn":
            p = deg[rows].astype(np.float32) * deg[ci].astype(np.float32)
            w = np.where(p > 0, np.float32(1.0) / np.sqrt(p, dtype=np.float32), np.float32(0.0)).astype(np.float32)
            return w.astype(dtype)
        t = np.dtype(dtype).type
        return (deg[rows].astype(t) * deg[ci].astype(t)).astype(dtype)
