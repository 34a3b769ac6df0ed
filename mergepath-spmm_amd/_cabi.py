"""ctypes binding of libmpspmm.so (include/mpspmm.h).

The library is the product; there is no Python or CPU fallback.  If the
shared object has not been built, loading raises and every operation fails.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmpspmm.so")

MPS_OK = 0
MPS_ERR_INVALID_ARG = 1
MPS_ERR_UNSUPPORTED = 2
MPS_ERR_WORKSPACE = 3
MPS_ERR_ALIGNMENT = 4
MPS_ERR_IO = 5
MPS_ERR_FORMAT = 6
MPS_ERR_TPW = 7
MPS_ERR_INVALID_CSR = 8
MPS_ERR_UNSORTED = 9
MPS_ERR_HIP = 1000

MPS_PHASE_MAIN = 1
MPS_PHASE_FIXUP = 2
MPS_PHASE_REDUCE = 4
MPS_PHASE_PREPARE = 8
MPS_WEIGHT_DEGREE_PRODUCT = 0
MPS_WEIGHT_GCN = 1
MPS_PLAN_NO_TILING = 1
MPS_PLAN_FORCE_TILING = 2
MPS_PLAN_NO_HOT = 4
MPS_PLAN_FORCE_HOT = 8
MPS_PLAN_NO_ROWBLOCK = 16
MPS_PLAN_FORCE_ROWBLOCK = 32
MPS_PLAN_NO_SOURCES = 64
MPS_PLAN_NO_ROW_MARKS = 128
MPS_PLAN_NO_RESIDENT = 256
MPS_PLAN_NO_COLUMN_TILES = 512
MPS_PLAN_LOCAL_TABLES = 1024
MPS_PLAN_NO_SWEEP = 2048
MPS_PLAN_FORCE_SWEEP = 4096
MPS_PLAN_HOST_BUILD = 8192
(MPS_PLAN_ARRAY_VROW_PTR, MPS_PLAN_ARRAY_COORD_X, MPS_PLAN_ARRAY_COORD_Y, MPS_PLAN_ARRAY_WAVE_OFF,
 MPS_PLAN_ARRAY_SLICE_COLS, MPS_PLAN_ARRAY_SLICE_SRC, MPS_PLAN_ARRAY_SLICE_VALS, MPS_PLAN_ARRAY_HOT_COLS,
 MPS_PLAN_ARRAY_RB_BLOCK_ROW, MPS_PLAN_ARRAY_RB_HOT_COLS, MPS_PLAN_ARRAY_RB_META, MPS_PLAN_ARRAY_RB_WAVE_BASE,
 MPS_PLAN_ARRAY_RB_HOT, MPS_PLAN_ARRAY_RB_COLD, MPS_PLAN_ARRAY_RB_HOT_SRC, MPS_PLAN_ARRAY_RB_COLD_SRC,
 MPS_PLAN_ARRAY_RB_HOT_PACKED, MPS_PLAN_ARRAY_RB_COLD_PACKED, MPS_PLAN_ARRAY_RB_COLD_BEGIN,
 MPS_PLAN_ARRAY_RB_TABLE_BASE, MPS_PLAN_ARRAY_SW_PANEL_PTR, MPS_PLAN_ARRAY_SW_ROWS, MPS_PLAN_ARRAY_SW_PIECE_PTR,
 MPS_PLAN_ARRAY_SW_WAVE_META, MPS_PLAN_ARRAY_SW_PANEL_ROUNDS, MPS_PLAN_ARRAY_SW_STREAM, MPS_PLAN_ARRAY_SW_SRC,
 MPS_PLAN_ARRAY_SW_SPLIT_ROW, MPS_PLAN_ARRAY_SW_SPLIT_PTR) = range(29)


class PlanInfo(ctypes.Structure):
    """struct mps_plan_info"""
    _fields_ = [(n, ctypes.c_int) for n in ("n_rows", "nnz", "K", "elem_bytes", "cost", "threads_per_wave",
                                             "num_slabs", "slab_cols", "num_partitions", "num_waves")] + \
               [("total_rounds", ctypes.c_longlong), ("slice_slots", ctypes.c_longlong),
                ("device_bytes", ctypes.c_size_t), ("num_segments", ctypes.c_int), ("hot_rows", ctypes.c_int),
                ("hot_waves", ctypes.c_int), ("hot_nnz", ctypes.c_longlong), ("hot_cost", ctypes.c_int), ("mark_shift", ctypes.c_int),
                ("hot_mark_shift", ctypes.c_int), ("hot_blocks", ctypes.c_int),
                ("rowblock_steps", ctypes.c_int), ("rowblock_table_rows", ctypes.c_int),
                ("rowblock_blocks", ctypes.c_int), ("rowblock_acc_rows", ctypes.c_int),
                ("rowblock_hot_slots", ctypes.c_longlong), ("rowblock_cold_slots", ctypes.c_longlong),
                ("resident_cols", ctypes.c_int), ("resident_nnz", ctypes.c_longlong),
                ("rowblock_cold_index_bits", ctypes.c_int), ("rowblock_local_tables", ctypes.c_int)] + \
               [(n, ctypes.c_int) for n in ("sweep_panels", "sweep_acc_rows", "sweep_lanes", "sweep_tiles", "sweep_col_bits",
                                             "sweep_piece", "sweep_together", "sweep_split_rows", "sweep_partial_rows", "sweep_listed_rows")] + \
               [("sweep_rounds", ctypes.c_longlong), ("sweep_slots", ctypes.c_longlong), ("built_on_device", ctypes.c_int)]


class PlanOptions(ctypes.Structure):
    """struct mps_plan_options"""
    _fields_ = [("flags", ctypes.c_uint), ("slab_bytes", ctypes.c_size_t), ("rowblock_steps", ctypes.c_int),
                ("rowblock_table_rows", ctypes.c_int), ("rowblock_block_rows", ctypes.c_int),
                ("rowblock_blocks_per_round", ctypes.c_int), ("degree_weights", ctypes.c_int),
                ("resident_bytes", ctypes.c_size_t), ("sweep_piece", ctypes.c_int), ("sweep_acc_rows", ctypes.c_int),
                ("sweep_panels_per_round", ctypes.c_int), ("sweep_together", ctypes.c_int)]


class TuneResult(ctypes.Structure):
    """struct mps_tune_result"""
    _fields_ = [("cost", ctypes.c_int), ("threads_per_wave", ctypes.c_int), ("flags", ctypes.c_uint),
                ("ms", ctypes.c_float), ("slab_bytes", ctypes.c_ulonglong)]

c_int_p = ctypes.POINTER(ctypes.c_int)
_vp, _i, _sz, _u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_uint64

# name -> (restype, argtypes); one entry per declaration in include/mpspmm.h
PROTOTYPES = {
    "mps_status_string": (ctypes.c_char_p, [_i]),
    "mps_version": (ctypes.c_char_p, []),
    "mps_num_partitions": (_i, [_i, _i, _i, c_int_p]),
    "mps_default_cost": (_i, [_i, _i, _i, _i, c_int_p]),
    "mps_items_per_partition": (_i, [_i, _i, _i, c_int_p]),
    "mps_max_threads_per_wave": (_i, [_i, _i, c_int_p]),
    "mps_csr_read_header": (_i, [ctypes.c_char_p, c_int_p, c_int_p]),
    "mps_csr_read": (_i, [ctypes.c_char_p, _i, _i, _vp, _vp]),
    "mps_csr_write": (_i, [ctypes.c_char_p, _i, _vp, _vp]),
    "mps_graph_generate": (_i, [ctypes.c_char_p, _u64, ctypes.POINTER(_vp)]),
    "mps_graph_from_edges": (_i, [_vp, _vp, ctypes.c_int64, ctypes.POINTER(_vp)]),
    "mps_graph_from_csr_file": (_i, [ctypes.c_char_p, ctypes.POINTER(_vp)]),
    "mps_graph_dims": (_i, [_vp, c_int_p, c_int_p, c_int_p]),
    "mps_graph_row_ptr": (_vp, [_vp]),
    "mps_graph_col_idx": (_vp, [_vp]),
    "mps_graph_free": (None, [_vp]),
    "mps_fill_uniform_f32": (_i, [_vp, _sz, _u64, ctypes.c_float, ctypes.c_float]),
    "mps_fill_uniform_f16": (_i, [_vp, _sz, _u64, ctypes.c_float, ctypes.c_float]),
    "mps_plan_autotune": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, ctypes.POINTER(TuneResult),
                               ctypes.POINTER(TuneResult), c_int_p]),
    "mps_degree_values_f32": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "mps_degree_values_f16": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "mps_csr_validate": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "mps_partition": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
    "mps_partition_host": (_i, [_vp, _i, _i, _i, _vp, _vp]),
    "mps_schedule_legacy": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mps_spmm_workspace_bytes": (_i, [_i, _i, _i, _i, ctypes.POINTER(_sz)]),
    "mps_spmm_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _sz, _vp]),
    "mps_static_scratch_bytes": (_i, [ctypes.POINTER(_sz)]),
    "mps_spmm_f32_static": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp]),
    "mps_spmm_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _sz, _vp]),
    "mps_spmm_f32_phases": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _sz,
                                 ctypes.c_uint, _vp]),
    "mps_spmm_f16_phases": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _sz,
                                 ctypes.c_uint, _vp]),
    "mps_tile_shape": (_i, [_i, _i, _i, _i, _sz, c_int_p, c_int_p]),
    "mps_plan_create": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, ctypes.c_uint, _sz, _vp, ctypes.POINTER(_vp)]),
    "mps_plan_create_ex": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, ctypes.POINTER(PlanOptions), _vp,
                                ctypes.POINTER(_vp)]),
    "mps_rowblock_layout_build": (_i, [_vp, _vp, _vp, _i, _i, _i, ctypes.POINTER(PlanOptions), ctypes.POINTER(_vp)]),
    "mps_rowblock_layout_info": (_i, [_vp, _vp]),
    "mps_rowblock_layout_array": (_i, [_vp, _i, ctypes.POINTER(_vp), ctypes.POINTER(_sz)]),
    "mps_rowblock_layout_free": (None, [_vp]),
    "mps_sweep_layout_build": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, ctypes.POINTER(PlanOptions), ctypes.POINTER(_vp)]),
    "mps_sweep_layout_info": (_i, [_vp, _vp]),
    "mps_sweep_layout_array": (_i, [_vp, _i, ctypes.POINTER(_vp), ctypes.POINTER(_sz)]),
    "mps_sweep_layout_free": (None, [_vp]),
    "mps_plan_destroy": (None, [_vp]),
    "mps_plan_get_info": (_i, [_vp, _vp]),
    "mps_plan_set_values": (_i, [_vp, _vp, _vp]),
    "mps_plan_copy_array": (_i, [_vp, _i, _vp, _sz]),
    "mps_plan_spmm_f32": (_i, [_vp, _vp, _vp, _vp]),
    "mps_plan_spmm_f16": (_i, [_vp, _vp, _vp, _vp]),
    "mps_plan_spmm_phases": (_i, [_vp, _vp, _vp, ctypes.c_uint, _vp]),
    "mps_rowwise_spmm_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mps_rowwise_bounds": (_i, [_i, _i, _vp, _vp]),
    "mps_nzsplit_max_parts": (_i, [_i, _i, _i, c_int_p]),
    "mps_nzsplit_build": (_i, [_vp, _i, _i, _vp, _vp, _i, _vp, c_int_p, _vp]),
    "mps_nzsplit_spmm_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp]),
}


class MpsError(RuntimeError):
    """A C-ABI call returned a non-zero mps_status."""

    def __init__(self, status, what=""):
        self.status = int(status)
        text = _lib.mps_status_string(self.status).decode() if _lib is not None else "?"
        if self.status >= MPS_ERR_HIP:
            text += " (hipError_t %d)" % (self.status - MPS_ERR_HIP)
        super().__init__("%s: mps_status %d: %s" % (what or "libmpspmm", self.status, text))


_lib = None


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmpspmm.so is not built (%s): run `make -C mergepath-spmm_amd/csrc` or "
                "__graft_entry__.build(); there is no fallback path" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status, what=""):
    if status != MPS_OK:
        raise MpsError(status, what)
