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

def default_cost(n_rows, nnz, K=16, elem_bytes=4):
    """Merge items (row ends + nonzeros) per partition when the caller gives no cost."""
    c = ctypes.c_int()
    check(_cabi.lib().mps_default_cost(int(n_rows), int(nnz), int(K), int(elem_bytes), ctypes.byref(c)), "mps_default_cost")
    return c.value


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


def autotune(csr, X, repeats=5):
    """Sweeps cost, partitions per wavefront and the plan switches for one
    matrix and K (mps_plan_autotune) - the sweep the reference's users run by
    hand over its <cost> and <threads_per_warp> arguments
    (src/MergePathSpMM.cu:121-122).  Returns (best, tried): dicts with cost,
    threads_per_wave, flags, ms, slab_bytes."""
    K = X.shape[1]
    eb = 4 if csr.val.dtype == torch.float32 else 2
    Y = torch.empty_like(X)
    best = _cabi.TuneResult()
    tried = (_cabi.TuneResult * 32)()
    n = ctypes.c_int(32)
    check(_cabi.lib().mps_plan_autotune(_ptr(csr.row_ptr), _ptr(csr.col_idx), _ptr(csr.val), csr.n_rows, csr.nnz, int(K),
                                        eb, _ptr(X), _ptr(Y), int(repeats), _stream(), ctypes.byref(best), tried,
                                        ctypes.byref(n)), "mps_plan_autotune")
    as_dict = lambda r: {"cost": r.cost, "threads_per_wave": r.threads_per_wave, "flags": r.flags, "ms": r.ms,
                         "slab_bytes": r.slab_bytes}
    return as_dict(best), [as_dict(tried[i]) for i in range(min(n.value, 32))]


def degree_values(row_ptr, col_idx, mode="product", dtype=torch.float32):
    """Edge weights from degrees on the device (mps_degree_values_*): the
    reference's implicit weight deg(row) * deg(col)
    (src/MergePathSpMM.cu:183-185,450,459) as an explicit value array, or the
    GCN normalisation 1 / sqrt(deg(row) * deg(col)) with mode="gcn"."""
    m = {"product": _cabi.MPS_WEIGHT_DEGREE_PRODUCT, "gcn": _cabi.MPS_WEIGHT_GCN}[mode]
    n_rows, nnz = row_ptr.numel() - 1, col_idx.numel()
    val = torch.empty(nnz, dtype=dtype, device=row_ptr.device)
    fn = _cabi.lib().mps_degree_values_f32 if dtype == torch.float32 else _cabi.lib().mps_degree_values_f16
    check(fn(_ptr(row_ptr), _ptr(col_idx), n_rows, nnz, m, _ptr(val), _stream()), "mps_degree_values")
    return val


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


def generate_mp_sched(row_ptr, nnz, cost=None, P=None, K=16, elem_bytes=4):
    """Merge-path split of (row_ptr, 0..nnz-1) into P partitions, on the device.  Without cost or P the
    library's default cost for feature width K and element size elem_bytes is used."""
    _need(row_ptr, torch.int32, "row_ptr")
    n_rows = int(row_ptr.numel()) - 1
    if P is None:
        P = num_partitions(n_rows, nnz, default_cost(n_rows, nnz, K, elem_bytes) if cost is None else cost)
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


def tile_shape(n_rows, nnz, K, elem_bytes=4, slab_bytes=0):
    ns, sc = ctypes.c_int(), ctypes.c_int()
    check(_cabi.lib().mps_tile_shape(int(n_rows), int(nnz), int(K), int(elem_bytes), int(slab_bytes),
                                     ctypes.byref(ns), ctypes.byref(sc)), "mps_tile_shape")
    return ns.value, sc.value


class Plan:
    """Per-matrix preprocessing (mps_plan_create): optional column-slab tiling,
    the merge-path partition of the (virtual) rows, the sliced nonzero arrays
    and the workspace.  The counterpart of what the reference sets up once
    before its repeat loop (src/MergePathSpMM.cu:192-220)."""

    def __init__(self, csr, K, cost=None, threads_per_wave=0, tiling="auto", slab_bytes=0, hot="auto",
                 rowblock="auto", rowblock_steps=0, rowblock_table_rows=0, rowblock_block_rows=0,
                 rowblock_blocks_per_round=0, keep_sources=True, row_marks=True, resident="auto", resident_bytes=0, weights=None, column_tiles=True,
                 local_tables=False, sweep="auto", sweep_piece=0, sweep_acc_rows=0, sweep_panels_per_round=0,
                 sweep_together=0, host_build=False):
        import numpy as np
        self._np = np
        self._h = ctypes.c_void_p()
        self.dtype = csr.val.dtype
        eb = 4 if self.dtype == torch.float32 else 2
        flags = {"auto": 0, "off": _cabi.MPS_PLAN_NO_TILING, "force": _cabi.MPS_PLAN_FORCE_TILING}[tiling]
        flags |= {"auto": 0, "off": _cabi.MPS_PLAN_NO_HOT, "force": _cabi.MPS_PLAN_FORCE_HOT}[hot]
        flags |= {"auto": 0, "off": _cabi.MPS_PLAN_NO_ROWBLOCK, "force": _cabi.MPS_PLAN_FORCE_ROWBLOCK}[rowblock]
        flags |= {"auto": 0, "off": _cabi.MPS_PLAN_NO_SWEEP, "force": _cabi.MPS_PLAN_FORCE_SWEEP}[sweep]
        if not keep_sources:
            flags |= _cabi.MPS_PLAN_NO_SOURCES
        if not row_marks:
            flags |= _cabi.MPS_PLAN_NO_ROW_MARKS
        if resident == "off":
            flags |= _cabi.MPS_PLAN_NO_RESIDENT
        if not column_tiles:
            flags |= _cabi.MPS_PLAN_NO_COLUMN_TILES
        if local_tables:
            flags |= _cabi.MPS_PLAN_LOCAL_TABLES
        if host_build:
            flags |= _cabi.MPS_PLAN_HOST_BUILD
        opt = _cabi.PlanOptions(flags, int(slab_bytes), int(rowblock_steps), int(rowblock_table_rows),
                                int(rowblock_block_rows), int(rowblock_blocks_per_round),
                                {None: 0, "degree": 1, "gcn": 2}[weights], int(resident_bytes), int(sweep_piece),
                                int(sweep_acc_rows), int(sweep_panels_per_round), int(sweep_together))
        check(_cabi.lib().mps_plan_create_ex(_ptr(csr.row_ptr), _ptr(csr.col_idx), None if weights else _ptr(csr.val),
                                             csr.n_rows, csr.nnz,
                                             int(K), eb, int(default_cost(csr.n_rows, csr.nnz, K, eb) if cost is None else cost),
                                             int(threads_per_wave), ctypes.byref(opt), _stream(),
                                             ctypes.byref(self._h)), "mps_plan_create_ex")
        self.K, self.n_rows = int(K), csr.n_rows
        info = _cabi.PlanInfo()
        check(_cabi.lib().mps_plan_get_info(self._h, ctypes.byref(info)), "mps_plan_get_info")
        self.info = info

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value and _cabi is not None:
            _cabi.lib().mps_plan_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_values(self, val):
        """The nonzero values changed, the pattern did not."""
        _need(val, self.dtype, "val")
        check(_cabi.lib().mps_plan_set_values(self._h, _ptr(val), _stream()), "mps_plan_set_values")

    def array(self, which):
        """Host copy of one of the plan's device arrays (numpy)."""
        np, i = self._np, self.info
        slots = int(i.slice_slots)
        shapes = {
            _cabi.MPS_PLAN_ARRAY_VROW_PTR: (i.num_segments * i.n_rows + 1, np.int32),
            _cabi.MPS_PLAN_ARRAY_COORD_X: (i.num_partitions + 1, np.int32),
            _cabi.MPS_PLAN_ARRAY_COORD_Y: (i.num_partitions + 1, np.int32),
            _cabi.MPS_PLAN_ARRAY_WAVE_OFF: (i.num_waves + 1, np.int32),
            _cabi.MPS_PLAN_ARRAY_SLICE_COLS: (slots, np.int32),
            _cabi.MPS_PLAN_ARRAY_SLICE_SRC: (slots, np.int32),
            _cabi.MPS_PLAN_ARRAY_SLICE_VALS: (slots, np.float32 if i.elem_bytes == 4 else np.float16),
            _cabi.MPS_PLAN_ARRAY_HOT_COLS: (i.num_slabs * i.hot_rows, np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_BLOCK_ROW: (i.rowblock_blocks + 1, np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_HOT_COLS: (i.rowblock_steps * i.rowblock_table_rows, np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_META: (i.rowblock_blocks * i.rowblock_steps * 64, np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_WAVE_BASE: (i.rowblock_blocks * 32, np.int64),
            _cabi.MPS_PLAN_ARRAY_RB_HOT: (0, np.uint32),  # host layouts only
            _cabi.MPS_PLAN_ARRAY_RB_COLD: (0 if i.rowblock_cold_index_bits else 2 * int(i.rowblock_cold_slots), np.uint32),
            _cabi.MPS_PLAN_ARRAY_RB_HOT_SRC: (int(i.rowblock_hot_slots), np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_COLD_SRC: (int(i.rowblock_cold_slots), np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_HOT_PACKED: (3 * int(i.rowblock_hot_slots) // 2, np.uint32),
            _cabi.MPS_PLAN_ARRAY_RB_COLD_PACKED: (3 * int(i.rowblock_cold_slots) // 2 if i.rowblock_cold_index_bits else 0, np.uint32),
            _cabi.MPS_PLAN_ARRAY_RB_COLD_BEGIN: (i.rowblock_steps + 1 if i.rowblock_steps else 0, np.int32),
            _cabi.MPS_PLAN_ARRAY_RB_TABLE_BASE: (i.rowblock_blocks if i.rowblock_local_tables else 0, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_PANEL_PTR: (i.sweep_panels + 1 if i.sweep_panels else 0, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_ROWS: (i.sweep_listed_rows, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_PIECE_PTR: (i.sweep_listed_rows + i.sweep_panels, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_WAVE_META: (i.sweep_panels * 32, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_PANEL_ROUNDS: (i.sweep_panels, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_STREAM: (2 * int(i.sweep_slots), np.uint32),
            _cabi.MPS_PLAN_ARRAY_SW_SRC: (int(i.sweep_slots), np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_SPLIT_ROW: (i.sweep_split_rows, np.int32),
            _cabi.MPS_PLAN_ARRAY_SW_SPLIT_PTR: (i.sweep_split_rows + 1 if i.sweep_panels else 0, np.int32),
        }
        n, dt = shapes[which]
        out = np.empty(n, dtype=dt)
        check(_cabi.lib().mps_plan_copy_array(self._h, int(which), out.ctypes.data, out.nbytes), "mps_plan_copy_array")
        return out

    def spmm(self, X, out=None, phases=None):
        """Y = A @ X."""
        _need(X, self.dtype, "X")
        if X.dim() != 2 or X.shape[0] != self.n_rows or X.shape[1] != self.K:
            raise ValueError("X must be [n_rows, K] with the K the plan was made for")
        Y = out if out is not None else torch.empty_like(X)
        _need(Y, self.dtype, "out")
        L = _cabi.lib()
        if phases is None:
            fn = L.mps_plan_spmm_f32 if self.dtype == torch.float32 else L.mps_plan_spmm_f16
            check(fn(self._h, _ptr(X), _ptr(Y), _stream()), "mps_plan_spmm")
        else:
            check(L.mps_plan_spmm_phases(self._h, _ptr(X), _ptr(Y), int(phases), _stream()), "mps_plan_spmm_phases")
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


class RowBlockLayout:
    """The layout of a row-block plan, built on the host (mps_rowblock_layout_build): no GPU needed."""

    def __init__(self, row_ptr, col_idx, val, K=16, steps=0, table_rows=0, block_rows=0, blocks_per_round=0,
                 keep_sources=True, local_tables=False):
        import numpy as np
        self._np = np
        self._h = ctypes.c_void_p()
        rp = np.ascontiguousarray(row_ptr, dtype=np.int32)
        ci = np.ascontiguousarray(col_idx, dtype=np.int32)
        v = np.ascontiguousarray(val, dtype=np.float32)
        opt = _cabi.PlanOptions((0 if keep_sources else _cabi.MPS_PLAN_NO_SOURCES) | (_cabi.MPS_PLAN_LOCAL_TABLES if local_tables else 0),
                                0, int(steps), int(table_rows),
                                int(block_rows), int(blocks_per_round), 0, 0, 0, 0, 0, 0)
        check(_cabi.lib().mps_rowblock_layout_build(rp.ctypes.data, ci.ctypes.data, v.ctypes.data, rp.size - 1, ci.size,
                                                    int(K), ctypes.byref(opt), ctypes.byref(self._h)),
              "mps_rowblock_layout_build")
        self.info = _cabi.PlanInfo()
        check(_cabi.lib().mps_rowblock_layout_info(self._h, ctypes.byref(self.info)), "mps_rowblock_layout_info")

    def array(self, which, dtype):
        """Copy of one of the layout's arrays (MPS_PLAN_ARRAY_RB_*) as a numpy array of `dtype`."""
        np = self._np
        data, nbytes = ctypes.c_void_p(), ctypes.c_size_t()
        check(_cabi.lib().mps_rowblock_layout_array(self._h, int(which), ctypes.byref(data), ctypes.byref(nbytes)),
              "mps_rowblock_layout_array")
        if nbytes.value == 0:
            return np.zeros(0, dtype=dtype)
        buf = (ctypes.c_char * nbytes.value).from_address(data.value)
        return np.frombuffer(buf, dtype=dtype).copy()

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            _cabi.lib().mps_rowblock_layout_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SweepLayout:
    """The layout of a sweep plan, built on the host (mps_sweep_layout_build): no GPU needed."""

    def __init__(self, row_ptr, col_idx, val, K, elem_bytes=4, piece=0, acc_rows=0, panels_per_round=0, keep_sources=True,
                 together=0):
        import numpy as np
        self._np = np
        self._h = ctypes.c_void_p()
        rp = np.ascontiguousarray(row_ptr, dtype=np.int32)
        ci = np.ascontiguousarray(col_idx, dtype=np.int32)
        v = np.ascontiguousarray(val, dtype=np.float32)
        opt = _cabi.PlanOptions(0 if keep_sources else _cabi.MPS_PLAN_NO_SOURCES, 0, 0, 0, 0, 0, 0, 0, int(piece), int(acc_rows),
                                int(panels_per_round), int(together))
        check(_cabi.lib().mps_sweep_layout_build(rp.ctypes.data, ci.ctypes.data, v.ctypes.data, rp.size - 1, ci.size, int(K),
                                                 int(elem_bytes), ctypes.byref(opt), ctypes.byref(self._h)),
              "mps_sweep_layout_build")
        self.info = _cabi.PlanInfo()
        check(_cabi.lib().mps_sweep_layout_info(self._h, ctypes.byref(self.info)), "mps_sweep_layout_info")

    def array(self, which, dtype):
        """Copy of one of the layout's arrays (MPS_PLAN_ARRAY_SW_*) as a numpy array of `dtype`."""
        np = self._np
        data, nbytes = ctypes.c_void_p(), ctypes.c_size_t()
        check(_cabi.lib().mps_sweep_layout_array(self._h, int(which), ctypes.byref(data), ctypes.byref(nbytes)),
              "mps_sweep_layout_array")
        if nbytes.value == 0:
            return np.zeros(0, dtype=dtype)
        buf = (ctypes.c_char * nbytes.value).from_address(data.value)
        return np.frombuffer(buf, dtype=dtype).copy()

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            _cabi.lib().mps_sweep_layout_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
