"""ctypes loader for libmatxtract_hip.so (the C ABI declared in include/matxtract_hip.h).

The library is built in-tree by ``matxtractt_amd/csrc/Makefile``.  Loading fails loudly when it
is missing: there is no Python or CPU fallback for the device entry points.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmatxtract_hip.so")
CSRC = os.path.join(_HERE, "csrc")

MX_OK, MX_ERR_ARG, MX_ERR_ALLOC, MX_ERR_DEVICE, MX_ERR_IO = 0, 1, 2, 3, 4
MX_F64, MX_F16 = 0, 1
MX_PLAN_DEFAULT, MX_PLAN_NO_TILES, MX_PLAN_ALL_TILES = 0, 1, 2
MX_PLAN_CSR_ROWS, MX_PLAN_CSR_SLICES, MX_PLAN_KEEP_TILES, MX_PLAN_NO_FUSE, MX_PLAN_FUSE = 4, 8, 16, 32, 64
MX_PLAN_KEEP, MX_PLAN_STREAM = 128, 256
MX_OPT_CSR_KEEP = 512
# mx_plan_info.opt_flags: the switches of the environment a plan was made under
MX_OPT_NO_STRIPS, MX_OPT_NO_BLOCKS, MX_OPT_NO_DICT, MX_OPT_STRIPS_APART, MX_OPT_CSR_KERNEL = 1, 2, 4, 8, 16
MX_OPT_CSR_FUSED, MX_OPT_AUTOTUNE, MX_OPT_LAYOUT_HOST, MX_OPT_TUNING = 32, 64, 128, 256


class MxError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("matxtract_hip error %d: %s" % (code, msg))
        self.code = code


class CsrStruct(C.Structure):
    _fields_ = [("rows", C.c_int), ("cols", C.c_int), ("nnz", C.c_int), ("dtype", C.c_int),
                ("rowPtr", C.c_void_p), ("colInd", C.c_void_p), ("val", C.c_void_p)]


class PartitionView(C.Structure):
    _fields_ = [
        ("dtype", C.c_int), ("rows", C.c_int), ("cols", C.c_int), ("nnz", C.c_int),
        ("fragM", C.c_int), ("fragK", C.c_int),
        ("dCols", C.c_int), ("sCols", C.c_int), ("nnzColD", C.c_int), ("nnzColS", C.c_int),
        ("dRows", C.c_int), ("sRows", C.c_int), ("nnzRowD", C.c_int), ("nnzRowS", C.c_int),
        ("cols_ratio", C.c_float), ("tc_nnz_ratio", C.c_double),
        ("descColId", C.c_void_p), ("newArray", C.c_void_p), ("rId", C.c_void_p),
        ("newArray_", C.c_void_p),
        ("ddRowPtr", C.c_void_p), ("ddColInd", C.c_void_p), ("ddVal", C.c_void_p),
        ("chunkNum", C.c_int), ("totalTcFrags", C.c_int), ("tcValCount", C.c_int),
        ("chunkPtr", C.c_void_p), ("sparse_AToX_index", C.c_void_p), ("fragPtr", C.c_void_p),
        ("fragBit", C.c_void_p), ("tcVal", C.c_void_p),
        ("nnzCD", C.c_int),
        ("cdRowPtr", C.c_void_p), ("cdColInd", C.c_void_p), ("cdVal", C.c_void_p),
        ("tau_c", C.c_float), ("tau_r", C.c_float),
    ]


class PlanInfo(C.Structure):
    _fields_ = [("dtype", C.c_int), ("rows", C.c_int), ("cols", C.c_int), ("nnz", C.c_int),
                ("tile_chunks", C.c_int), ("tile_frags", C.c_int), ("tile_nnz", C.c_int),
                ("csr_nnz", C.c_int), ("csr_blocks", C.c_int), ("csr_variant", C.c_int),
                ("tile_bytes", C.c_double), ("csr_bytes", C.c_double),
                ("csr_main_kernel", C.c_int), ("csr_main_nnz", C.c_int), ("tile_variant", C.c_int), ("tile_strip_nnz", C.c_int),
                ("csr_value_dict", C.c_int), ("est_rows_us", C.c_double), ("est_slices_us", C.c_double),
                ("prep_route", C.c_int), ("ext_dCols", C.c_int), ("ext_dRows", C.c_int), ("ext_nnzRowD", C.c_int),
                ("ext_frags", C.c_int), ("csr_fused", C.c_int), ("opt_flags", C.c_int), ("opt_tile_gate", C.c_double), ("csr_keep", C.c_int), ("touched_bytes", C.c_double)]


class TauEstimate(C.Structure):
    _fields_ = [("tau_c", C.c_float), ("tau_r", C.c_float), ("saved_us", C.c_double), ("tile_entries", C.c_longlong)]


class TileStepsView(C.Structure):
    _fields_ = [("steps", C.c_int), ("nWaves", C.c_int), ("totalBlocks", C.c_longlong), ("stepDesc", C.c_void_p),
                ("chunkBlock0", C.c_void_p), ("waveDesc", C.c_void_p)]


class PlanArray(C.Structure):
    _fields_ = [("name", C.c_char_p), ("bytes", C.c_size_t), ("data", C.c_void_p)]


class SliceLayoutView(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("nWG", "S", "sliceCols", "waves", "stepEntries", "batchEntries", "cap", "chunks",
                                       "batches", "vrows", "nLight", "nHeavy", "lightSegs")] + \
               [("nEcol", C.c_longlong)] + \
               [(n, C.c_void_p) for n in ("wgDesc", "waveDesc", "chunkEnd", "segPtr", "segIdx", "rowInfo", "lightInfo",
                                        "heavyInfo", "ecol", "eval")] + \
               [("nDict", C.c_int), ("ecode", C.c_void_p), ("dict", C.c_void_p)] + \
               [(n, C.c_int) for n in ("fused", "groupRows", "nGroups", "placesPerRow")] + \
               [(n, C.c_void_p) for n in ("wgGroups", "groupNeed", "fusedTarget", "rowVrows")]


class TileLayoutView(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("steps", "nWaves", "chunks", "nnz", "dense")] + [("nVal", C.c_longlong)] + \
               [(n, C.c_void_p) for n in ("hdr", "atox", "waveDesc", "valOffset", "val")]


class PlanLayoutView(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("rows", "cols", "csr_nnz", "fragM", "fragK", "slots")] + \
               [(n, C.c_void_p) for n in ("csrRowPtr", "csrColInd", "csrVal", "stripRows")] + \
               [("tiles", TileLayoutView * 2), ("csr_variant", C.c_int), ("est_rows_us", C.c_double),
                ("est_slices_us", C.c_double)]


class KernelTime(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("ms", C.c_double), ("algorithmic_bytes", C.c_double), ("nnz", C.c_int),
                ("reserved", C.c_int)]


class TauPoint(C.Structure):
    _fields_ = [("tau_c", C.c_float), ("tau_r", C.c_float), ("ms_total", C.c_double), ("tile_nnz", C.c_int)]


# Every symbol include/matxtract_hip.h declares: name -> (restype, argtypes)
_vp, _i, _d = C.c_void_p, C.c_int, C.c_double
_pp = C.POINTER(C.c_void_p)
_pi = C.POINTER(C.c_int)
_pd = C.POINTER(C.c_double)
class DeviceTiles(C.Structure):
    _fields_ = [("chunkNum", _i), ("totalTcFrags", _i), ("fragK", _i), ("tcValCount", _i), ("chunkPtr", _vp),
                ("sparse_AToX_index", _vp), ("fragPtr", _vp), ("fragBit", _vp), ("tcVal", _vp), ("base", _vp)]


SIGNATURES = {
    "mx_last_error": (C.c_char_p, []),
    "mx_partition_create": (_i, [C.POINTER(CsrStruct), C.c_float, C.c_float, _pp]),
    "mx_partition_create_device": (_i, [C.POINTER(CsrStruct), C.c_float, C.c_float, _pp]),
    "mx_partition_destroy": (None, [_vp]),
    "mx_partition_get": (_i, [_vp, C.POINTER(PartitionView)]),
    "mx_partition_counts": (_i, [_vp, C.POINTER(PartitionView)]),
    "mx_partition_hash": (C.c_uint64, [_vp]),
    "mx_partition_save": (_i, [_vp, C.c_char_p]),
    "mx_partition_load": (_i, [C.c_char_p, _i, _pp]),
    "mx_transpose": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _pp, _pp, _pp]),
    "mx_transpose_device": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mx_select_device": (_i, [_i, _i, _i, _vp, _vp, C.c_float, C.c_float, _vp, _vp, _vp, _vp]),
    "mx_split_device": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mx_tiles_device": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, C.POINTER(DeviceTiles), _vp]),
    "mx_tiles_device_free": (None, [C.POINTER(DeviceTiles)]),
    "mx_free": (None, [_vp]),
    "mx_mmio_read": (_i, [C.c_char_p, _i, _pi, _pi, _pi, _pi, _pp, _pp, _pp]),
    "mx_init_vec": (None, [_i, _vp, _i]),
    "mx_f32_to_f16": (C.c_uint16, [C.c_float]),
    "mx_f16_to_f32": (C.c_float, [C.c_uint16]),
    "mx_gen_config": (_i, [_i, C.c_uint64, _d, _pi, _pi, _pi, _pi, _pp, _pp, _pp, _pp]),
    "mx_gen_config_ex": (_i, [_i, C.c_uint64, _d, _i, _pi, _pi, _pi, _pi, _pp, _pp, _pp, _pp]),
    "mx_gen_config_family": (_i, [_i, C.c_uint64, _d, _i, _d, _pi, _pi, _pi, _pi, _pp, _pp, _pp, _pp]),
    "mx_algorithmic_bytes": (_d, [_i, _i, _i, _i]),
    "mx_plan_create": (_i, [_vp, _i, _pp]),
    "mx_plan_create_device_csr": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _i, _pp]),
    "mx_plan_create_device": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, C.c_float, C.c_float, _i, _pp]),
    "mx_estimate_tau": (_i, [_vp, _i, _vp, _vp, _vp, _i, _vp]),
    "mx_tile_steps": (_i, [_vp, _i, _i, _i, _i, _i, _vp]),
    "mx_tile_steps_free": (None, [_vp]),
    "mx_plan_arrays": (_i, [_vp, _vp, _i, _vp]),
    "mx_plan_arrays_free": (None, [_vp, _i]),
    "mx_plan_destroy": (None, [_vp]),
    "mx_spmv": (_i, [_vp, _vp, _vp, _vp]),
    "mx_spmv_static": (_i, [_vp, _vp, _vp, _vp]),
    "mx_static_scratch_bytes": (_i, []),
    "mx_spmv_repeat": (_i, [_vp, _vp, _vp, _i, _vp]),
    "mx_spmv_host": (_i, [_vp, _vp, _vp]),
    "mx_time": (_i, [_vp, _vp, _vp, _i, _i, _pd, _pd, _pd]),
    "mx_time_rotate": (_i, [_vp, _vp, _vp, _i, _i, _i, _pd]),
    "mx_time_kernels": (_i, [_vp, _vp, _vp, _i, _i, C.POINTER(KernelTime), _i, _pi]),
    "mx_time_csr_main": (_i, [_vp, _vp, _vp, _i, _i, _pd]),
    "mx_plan_get_info": (_i, [_vp, C.POINTER(PlanInfo)]),
    "mx_tune_tau": (_i, [C.POINTER(CsrStruct), _i, _i, _i, _i, C.POINTER(C.c_float), C.POINTER(C.c_float),
                         C.POINTER(TauPoint), _i, _pi]),
    "mx_slice_layout": (_i, [C.POINTER(CsrStruct), _i, _vp, C.POINTER(SliceLayoutView)]),
    "mx_slice_layout_device": (_i, [C.POINTER(CsrStruct), _i, C.POINTER(SliceLayoutView)]),
    "mx_slice_layout_fused": (_i, [C.POINTER(CsrStruct), _i, C.POINTER(SliceLayoutView)]),
    "mx_debug_fused_misplaced": (_i, [_i]),
    "mx_slice_layout_free": (None, [C.POINTER(SliceLayoutView)]),
    "mx_plan_layout": (_i, [_vp, _i, _i, C.POINTER(PlanLayoutView)]),
    "mx_plan_layout_free": (None, [C.POINTER(PlanLayoutView)]),
    "mx_cdspmv_f64": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _pd, _pd]),
    "mx_cdspmv_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _pd, _pd]),
    "mx_du_tcspmv_f64": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _pd]),
    "mx_du_tcspmv_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _pd]),
    "mx_device_count": (_i, []),
    "mx_probe_mfma_f64": (_i, [_vp, _vp, _vp]),
    "mx_probe_mfma_f16": (_i, [_vp, _vp, _vp]),
}

_lib = None


def load():
    """Load the shared library (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s not found: build it with `make -C %s` (or __graft_entry__.build())" % (LIB_PATH, CSRC))
        # PyTorch ships its own copy of the HIP runtime under the same soname; whichever copy
        # is loaded first serves the whole process.  Import torch first so that device memory
        # and streams handed over by torch belong to the runtime this library talks to.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc):
    if rc != MX_OK:
        raise MxError(rc, load().mx_last_error().decode("utf-8", "replace"))
