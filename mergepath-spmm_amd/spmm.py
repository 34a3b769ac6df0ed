"""Device-side operators on torch tensors, one per step of the reference programs.

torch is used for device memory and the current stream only; every
computation is a call through the C ABI (include/mpspmm.h).  Names follow the
reference: generate_mp_sched / spmm_merge_path (src/MergePathSpMM.cu),
run_spmm_row_wise (src/row_wise.cu), build_part / nz-splitting
(src/nz_splitting.cu).
"""
import ctypes

import torch

from . import _cabi
from ._cabi import check

# Merge items (row ends + nonzeros) per partition when the caller gives no cost.
DEFAULT_COST = 128


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _need(t, dtype, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA/HIP torch tensor" % name)
    if t.dtype != dtype:
        raise TypeError("%s must have dtype %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    return t


class CsrDevice:
    """CSR arrays resident in HBM: row_ptr int32[N+1], col_idx int32[nnz], val."""

    def __init__(self, row_ptr, col_idx, val):
        self.row_ptr = _need(row_ptr, torch.int32, "row_ptr")
        self.col_idx = _need(col_idx, torch.int32, "col_idx")
        if val.dtype not in (torch.float32, torch.float16):
            raise TypeError("val must be float32 or float16")
        self.val = _need(val, val.dtype, "val")
        self.n_rows = int(row_ptr.numel()) - 1
        self.nnz = int(col_idx.numel())
        if self.val.numel() != self.nnz:
            raise ValueError("val and col_idx differ in length")

    def validate(self):
        check(_cabi.lib().mps_csr_validate(_ptr(self.row_ptr), _ptr(self.col_idx), self.n_rows, self.n_rows,
                                           self.nnz, _stream()), "mps_csr_validate")


class MergePathSchedule:
    """Partition count and boundary coordinates (generate_mp_sched, :300-385)."""

    def __init__(self, P, coord_x, coord_y, n_rows, nnz):
        self.P, self.coord_x, self.coord_y = P, coord_x, coord_y
        self.n_rows, self.nnz = n_rows, nnz
        self._ws = {}

    def workspace(self, K, tpw, elem_bytes):
        key = (K, tpw, elem_bytes)
        if key not in self._ws:
            nbytes = ctypes.c_size_t()
            check(_cabi.lib().mps_spmm_workspace_bytes(self.P, K, tpw, elem_bytes, ctypes.byref(nbytes)),
                  "mps_spmm_workspace_bytes")
            self._ws[key] = torch.empty(max(int(nbytes.value), 16), dtype=torch.uint8, device=self.coord_x.device)
        return self._ws[key]

    def legacy_arrays(self, row_ptr):
        """The six int32[P] arrays of the reference schedule, in upload order (:209-220)."""
        out = [torch.empty(self.P, dtype=torch.int32, device=row_ptr.device) for _ in range(6)]
        check(_cabi.lib().mps_schedule_legacy(_ptr(row_ptr), self.n_rows, self.nnz, self.P, _ptr(self.coord_x),
                                              _ptr(self.coord_y), *[_ptr(o) for o in out], _stream()),
              "mps_schedule_legacy")
        names = ("feature_start", "feature_start_num", "feature_end", "feature_end_num", "start_row", "end_row")
        return dict(zip(names, out))


def num_partitions(n_rows, nnz, cost):
    p = ctypes.c_int()
    check(_cabi.lib().mps_num_partitions(int(n_rows), int(nnz), int(cost), ctypes.byref(p)), "mps_num_partitions")
    return p.value


def generate_mp_sched(row_ptr, nnz, cost=None, P=None):
    """Merge-path split of (row_ptr, 0..nnz-1) into P partitions, on the device."""
    _need(row_ptr, torch.int32, "row_ptr")
    n_rows = int(row_ptr.numel()) - 1
    if P is None:
        P = num_partitions(n_rows, nnz, DEFAULT_COST if cost is None else cost)
    cx = torch.empty(P + 1, dtype=torch.int32, device=row_ptr.device)
    cy = torch.empty(P + 1, dtype=torch.int32, device=row_ptr.device)
    check(_cabi.lib().mps_partition(_ptr(row_ptr), n_rows, int(nnz), int(P), _ptr(cx), _ptr(cy), _stream()),
          "mps_partition")
    return MergePathSchedule(int(P), cx, cy, n_rows, int(nnz))


def spmm_merge_path(csr, X, sched, threads_per_wave=0, out=None, phases=None):
    """Y = A @ X with the merge-path kernels; fp32 or fp16 by the dtype of X."""
    dtype = X.dtype
    if dtype not in (torch.float32, torch.float16) or csr.val.dtype != dtype:
        raise TypeError("X and val must both be float32 or both float16")
    _need(X, dtype, "X")
    if X.dim() != 2 or X.shape[0] != csr.n_rows:
        raise ValueError("X must be [n_rows, K]")
    K = int(X.shape[1])
    Y = out if out is not None else torch.empty_like(X)
    _need(Y, dtype, "out")
    eb = 4 if dtype == torch.float32 else 2
    ws = sched.workspace(K, threads_per_wave, eb)
    L = _cabi.lib()
    args = [_ptr(csr.row_ptr), _ptr(csr.col_idx), _ptr(csr.val), _ptr(X), _ptr(Y), csr.n_rows, csr.nnz, K,
            sched.P, _ptr(sched.coord_x), _ptr(sched.coord_y), int(threads_per_wave), _ptr(ws), ws.numel()]
    if phases is None:
        fn = L.mps_spmm_f32 if eb == 4 else L.mps_spmm_f16
        check(fn(*args, _stream()), "mps_spmm")
    else:
        fn = L.mps_spmm_f32_phases if eb == 4 else L.mps_spmm_f16_phases
        check(fn(*args, int(phases), _stream()), "mps_spmm_phases")
    return Y


class TiledCsr:
    """Column-slab tiled copy of a CSR matrix plus the merge-path schedule over
    its virtual rows (mps_tile_build; no counterpart in the reference)."""

    def __init__(self, csr, num_slabs, slab_cols, vrow_ptr, col_tiled, perm, val_tiled):
        self.n_rows, self.nnz = csr.n_rows, csr.nnz
        self.num_slabs, self.slab_cols = num_slabs, slab_cols
        self.vrow_ptr, self.col_tiled, self.perm, self.val_tiled = vrow_ptr, col_tiled, perm, val_tiled
        self.sched = None
        self._ws = {}

    def set_values(self, val):
        """Re-gather the tiled values after the caller changed val."""
        eb = 4 if val.dtype == torch.float32 else 2
        check(_cabi.lib().mps_tile_gather_values(_ptr(val), _ptr(self.perm), self.nnz, eb, _ptr(self.val_tiled),
                                                 _stream()), "mps_tile_gather_values")

    def workspace(self, K, tpw, elem_bytes):
        key = (K, tpw, elem_bytes)
        if key not in self._ws:
            nbytes = ctypes.c_size_t()
            check(_cabi.lib().mps_spmm_tiled_workspace_bytes(self.n_rows, self.num_slabs, self.sched.P, K, tpw,
                                                             elem_bytes, ctypes.byref(nbytes)),
                  "mps_spmm_tiled_workspace_bytes")
            self._ws[key] = torch.empty(max(int(nbytes.value), 16), dtype=torch.uint8, device=self.vrow_ptr.device)
        return self._ws[key]


def tile_shape(n_rows, nnz, K, elem_bytes=4, slab_bytes=0):
    ns, sc = ctypes.c_int(), ctypes.c_int()
    check(_cabi.lib().mps_tile_shape(int(n_rows), int(nnz), int(K), int(elem_bytes), int(slab_bytes),
                                     ctypes.byref(ns), ctypes.byref(sc)), "mps_tile_shape")
    return ns.value, sc.value


def build_tiles(csr, K, cost=None, slab_bytes=0, num_slabs=None, slab_cols=None):
    """Tile csr for feature width K and build the schedule over the virtual rows.
    Returns None when tiling does not pay for this shape (unless slabs are forced)."""
    eb = 4 if csr.val.dtype == torch.float32 else 2
    if num_slabs is None:
        num_slabs, slab_cols = tile_shape(csr.n_rows, csr.nnz, K, eb, slab_bytes)
        if num_slabs <= 1:
            return None
    dev = csr.row_ptr.device
    nv = num_slabs * csr.n_rows
    vrow_ptr = torch.empty(nv + 1, dtype=torch.int32, device=dev)
    col_tiled = torch.empty(max(csr.nnz, 1), dtype=torch.int32, device=dev)
    perm = torch.empty(max(csr.nnz, 1), dtype=torch.int32, device=dev)
    scratch = torch.empty(nv + 2049, dtype=torch.int32, device=dev)
    check(_cabi.lib().mps_tile_build(_ptr(csr.row_ptr), _ptr(csr.col_idx), csr.n_rows, csr.nnz, num_slabs, slab_cols,
                                     _ptr(vrow_ptr), _ptr(col_tiled), _ptr(perm), _ptr(scratch), _stream()),
          "mps_tile_build")
    del scratch
    val_tiled = torch.empty(max(csr.nnz, 1), dtype=csr.val.dtype, device=dev)
    t = TiledCsr(csr, num_slabs, slab_cols, vrow_ptr, col_tiled, perm, val_tiled)
    t.set_values(csr.val)
    t.sched = generate_mp_sched(vrow_ptr, csr.nnz, cost=cost)
    return t


def spmm_merge_path_tiled(tiled, X, threads_per_wave=0, out=None, phases=None):
    """Y = A @ X from the tiled arrays (mps_spmm_tiled_f32 / _f16)."""
    dtype = X.dtype
    if dtype not in (torch.float32, torch.float16) or tiled.val_tiled.dtype != dtype:
        raise TypeError("X and val must both be float32 or both float16")
    _need(X, dtype, "X")
    if X.dim() != 2 or X.shape[0] != tiled.n_rows:
        raise ValueError("X must be [n_rows, K]")
    K = int(X.shape[1])
    Y = out if out is not None else torch.empty_like(X)
    eb = 4 if dtype == torch.float32 else 2
    ws = tiled.workspace(K, threads_per_wave, eb)
    sched = tiled.sched
    L = _cabi.lib()
    args = [_ptr(tiled.vrow_ptr), _ptr(tiled.col_tiled), _ptr(tiled.val_tiled), _ptr(X), _ptr(Y), tiled.n_rows,
            tiled.nnz, K, tiled.num_slabs, sched.P, _ptr(sched.coord_x), _ptr(sched.coord_y), int(threads_per_wave),
            _ptr(ws), ws.numel()]
    if phases is None:
        fn = L.mps_spmm_tiled_f32 if eb == 4 else L.mps_spmm_tiled_f16
        check(fn(*args, _stream()), "mps_spmm_tiled")
    else:
        fn = L.mps_spmm_tiled_f32_phases if eb == 4 else L.mps_spmm_tiled_f16_phases
        check(fn(*args, int(phases), _stream()), "mps_spmm_tiled_phases")
    return Y


def run_spmm_row_wise(csr, X, num_waves, out=None):
    """Row-split comparison kernel (src/row_wise.cu:172-240), fp32."""
    _need(X, torch.float32, "X")
    K = int(X.shape[1])
    Y = out if out is not None else torch.empty_like(X)
    check(_cabi.lib().mps_rowwise_spmm_f32(_ptr(csr.row_ptr), _ptr(csr.col_idx), _ptr(csr.val), _ptr(X), _ptr(Y),
                                           csr.n_rows, csr.nnz, K, int(num_waves), _stream()),
          "mps_rowwise_spmm_f32")
    return Y


class NzParts:
    """Neighbour groups of the nz-splitting kernel (build_part, src/nz_splitting.cu:256-297)."""

    def __init__(self, part_ptr, part2node, num_parts, part_size):
        self.part_ptr, self.part2node = part_ptr, part2node
        self.num_parts, self.part_size = num_parts, part_size


def build_part(row_ptr, nnz, part_size):
    _need(row_ptr, torch.int32, "row_ptr")
    n_rows = int(row_ptr.numel()) - 1
    L = _cabi.lib()
    mp = ctypes.c_int()
    check(L.mps_nzsplit_max_parts(n_rows, int(nnz), int(part_size), ctypes.byref(mp)), "mps_nzsplit_max_parts")
    dev = row_ptr.device
    part_ptr = torch.empty(mp.value + 1, dtype=torch.int32, device=dev)
    part2node = torch.empty(max(mp.value, 1), dtype=torch.int32, device=dev)
    scratch = torch.empty(n_rows + 1 + 2048, dtype=torch.int32, device=dev)
    num = ctypes.c_int()
    check(L.mps_nzsplit_build(_ptr(row_ptr), n_rows, int(part_size), _ptr(part_ptr), _ptr(part2node), mp.value,
                              _ptr(scratch), ctypes.byref(num), _stream()), "mps_nzsplit_build")
    return NzParts(part_ptr[: num.value + 1], part2node[: num.value], num.value, int(part_size))


def spmm_nz_splitting(csr, X, parts, out=None):
    """Nonzero-splitting comparison kernel (src/nz_splitting.cu:212-240, :318-445), fp32."""
    _need(X, torch.float32, "X")
    K = int(X.shape[1])
    Y = out if out is not None else torch.empty_like(X)
    check(_cabi.lib().mps_nzsplit_spmm_f32(_ptr(csr.col_idx), _ptr(csr.val), _ptr(X), _ptr(Y), csr.n_rows,
                                           csr.nnz, K, _ptr(parts.part_ptr), _ptr(parts.part2node),
                                           parts.num_parts, _stream()), "mps_nzsplit_spmm_f32")
    return Y
