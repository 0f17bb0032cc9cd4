"""Python face of libmatxtract_hip.so: numpy in/out for the host calls, torch tensors (device
memory and streams only) for the device calls.  Every function forwards to one C-ABI entry
point; nothing is computed in Python.

Names follow the reference driver (test/test_autotc_spmv.cpp): a ``Partition`` is what its
main() derives from (A, col_frac, hot_frac); a ``Plan`` is that partition resident on the GPU.
"""
import ctypes as C
import os

import numpy as np

from . import _lib
from ._lib import (MX_F16, MX_F64, MX_PLAN_ALL_TILES, MX_PLAN_CSR_SLICES, MX_PLAN_CSR_ROWS, MX_PLAN_DEFAULT,
                   MX_PLAN_FUSE, MX_PLAN_KEEP, MX_PLAN_STREAM, MX_OPT_CSR_KEEP, MX_PLAN_KEEP_TILES, MX_PLAN_NO_FUSE, MX_PLAN_NO_TILES, MX_OPT_NO_STRIPS, MX_OPT_NO_BLOCKS,
                   MX_OPT_NO_DICT, MX_OPT_STRIPS_APART, MX_OPT_CSR_KERNEL, MX_OPT_CSR_FUSED, MX_OPT_AUTOTUNE,
                   MX_OPT_LAYOUT_HOST, MX_OPT_TUNING, MxError, check)

__all__ = ["Csr", "Partition", "Plan", "gen_config", "mmio_read", "transpose", "transpose_device", "select_device", "split_device", "tiles_device", "cdspmv",
           "du_tcspmv", "algorithmic_bytes", "device_count", "init_vec", "slice_layout", "tune_tau", "estimate_tau", "tile_steps", "MxError",
           "MX_F64", "MX_F16", "MX_PLAN_DEFAULT", "MX_PLAN_NO_TILES", "MX_PLAN_ALL_TILES", "MX_PLAN_CSR_ROWS",
           "MX_PLAN_CSR_SLICES", "MX_PLAN_KEEP_TILES", "MX_PLAN_NO_FUSE", "MX_PLAN_FUSE", "MX_PLAN_KEEP", "MX_PLAN_STREAM", "MX_OPT_CSR_KEEP", "time_rotate", "plan_layout", "debug_fused_misplaced",
           "MX_OPT_NO_STRIPS", "MX_OPT_NO_BLOCKS", "MX_OPT_NO_DICT", "MX_OPT_STRIPS_APART", "MX_OPT_CSR_KERNEL",
           "MX_OPT_CSR_FUSED", "MX_OPT_AUTOTUNE", "MX_OPT_LAYOUT_HOST", "MX_OPT_TUNING"]


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _np_dtype(dt):
    return np.float64 if dt == MX_F64 else np.float16


def _take(addr, n, dtype, free=True):
    """Copy n items from a malloc()ed C array into numpy, then release it."""
    dtype = np.dtype(dtype)
    if n > 0 and addr:
        buf = (C.c_char * (n * dtype.itemsize)).from_address(addr)
        out = np.frombuffer(buf, dtype=dtype, count=n).copy()
    else:
        out = np.zeros(0, dtype)
    if free and addr:
        _lib.load().mx_free(addr)
    return out


def _view(addr, n, dtype):
    return _take(addr, n, dtype, free=False)


def device_count():
    return _lib.load().mx_device_count()


def algorithmic_bytes(dtype, rows, cols, nnz):
    return _lib.load().mx_algorithmic_bytes(dtype, rows, cols, nnz)


class Csr:
    """The reference's CSR triple (csrVal, csrRowPtr, csrColInd) plus its shape."""

    def __init__(self, rows, cols, rowPtr, colInd, val):
        self.rows, self.cols = int(rows), int(cols)
        self.rowPtr = np.ascontiguousarray(rowPtr, dtype=np.int32)
        self.colInd = np.ascontiguousarray(colInd, dtype=np.int32)
        val = np.ascontiguousarray(val)
        if val.dtype == np.uint16:
            val = val.view(np.float16)
        if val.dtype not in (np.float64, np.float16):
            raise TypeError("values must be float64 or float16")
        self.val = val
        self.nnz = int(len(self.colInd))
        self.dtype = MX_F64 if val.dtype == np.float64 else MX_F16

    def struct(self):
        return _lib.CsrStruct(self.rows, self.cols, self.nnz, self.dtype, _p(self.rowPtr).value,
                              _p(self.colInd).value, _p(self.val).value)

    @property
    def algorithmic_bytes(self):
        return algorithmic_bytes(self.dtype, self.rows, self.cols, self.nnz)


def gen_config(config_id, seed=0, scale=1.0, unaligned=False, dense_share=None):
    """Synthetic workload 1..5 -> (Csr, x).  unaligned=True: the dense blocks of workload 2 and the strips of
    workload 5 start off the grid of eight columns (MX_GEN_UNALIGNED).  dense_share: how much of workload 2
    (share of the entries in 8x8 blocks, 0.4 in the benchmark) or 5 (probability that a run of 128 rows is a
    strip, 0.2) is dense structure (mx_gen_config_family)."""
    L = _lib.load()
    rows, cols, nnz, dt = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    rp, ci, va, xv = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(L.mx_gen_config_family(config_id, seed, scale, 1 if unaligned else 0, -1.0 if dense_share is None else float(dense_share),
                                 C.byref(rows), C.byref(cols), C.byref(nnz), C.byref(dt), C.byref(rp), C.byref(ci), C.byref(va),
                                 C.byref(xv)))
    vt = _np_dtype(dt.value)
    A = Csr(rows.value, cols.value, _take(rp.value, rows.value + 1, np.int32),
            _take(ci.value, nnz.value, np.int32), _take(va.value, nnz.value, vt))
    return A, _take(xv.value, cols.value, vt)


def mmio_read(path, dtype=MX_F64):
    L = _lib.load()
    rows, cols, nnz, sym = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    rp, ci, va = C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(L.mx_mmio_read(str(path).encode(), dtype, C.byref(rows), C.byref(cols), C.byref(nnz), C.byref(sym),
                         C.byref(rp), C.byref(ci), C.byref(va)))
    A = Csr(rows.value, cols.value, _take(rp.value, rows.value + 1, np.int32),
            _take(ci.value, nnz.value, np.int32), _take(va.value, nnz.value, _np_dtype(dtype)))
    return A, bool(sym.value)


def init_vec(n, dtype=MX_F64):
    v = np.zeros(n, _np_dtype(dtype))
    _lib.load().mx_init_vec(dtype, _p(v), n)
    return v


def transpose(ptr, ind, val, inner):
    """csr2csc / csc2csr: stable counting-sort transpose."""
    ptr = np.ascontiguousarray(ptr, dtype=np.int32)
    ind = np.ascontiguousarray(ind, dtype=np.int32)
    val = np.ascontiguousarray(val)
    dt = MX_F64 if val.dtype == np.float64 else MX_F16
    tp, ti, tv = C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(_lib.load().mx_transpose(dt, len(ptr) - 1, inner, len(ind), _p(ptr), _p(ind), _p(val),
                                   C.byref(tp), C.byref(ti), C.byref(tv)))
    return (_take(tp.value, inner + 1, np.int32), _take(ti.value, len(ind), np.int32),
            _take(tv.value, len(ind), val.dtype))


def transpose_device(ptr, ind, val, inner, stream=None):
    """csr2csc / csc2csr on the device: torch device tensors in (int32 ptr and ind, float64 or
    float16 val), torch device tensors out, same arrays as transpose()."""
    import torch
    for name, t, dt in (("ptr", ptr, torch.int32), ("ind", ind, torch.int32)):
        if (not t.is_cuda) or t.dtype != dt or not t.is_contiguous():
            raise ValueError("%s must be a contiguous int32 device tensor" % name)
    if (not val.is_cuda) or val.dtype not in (torch.float64, torch.float16) or not val.is_contiguous() \
            or val.numel() != ind.numel():
        raise ValueError("val must be a contiguous float64 or float16 device tensor as long as ind")
    dt = MX_F64 if val.dtype == torch.float64 else MX_F16
    nnz = ind.numel()
    tp = torch.empty(inner + 1, dtype=torch.int32, device=ptr.device)
    ti = torch.empty(nnz, dtype=torch.int32, device=ptr.device)
    tv = torch.empty(nnz, dtype=val.dtype, device=ptr.device)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    check(_lib.load().mx_transpose_device(dt, ptr.numel() - 1, inner, nnz, ptr.data_ptr(), ind.data_ptr(),
                                          val.data_ptr(), tp.data_ptr(), ti.data_ptr(), tv.data_ptr(), s))
    return tp, ti, tv


def select_device(rowPtr, colInd, cols, tau_c, tau_r, stream=None):
    """The column and row selections of the cascaded extraction on a device-resident CSR matrix:
    returns (descColId, descRowId, {dCols, nnzColD, dRows, nnzRowD}); the orders are device tensors."""
    import torch
    for name, t in (("rowPtr", rowPtr), ("colInd", colInd)):
        if (not t.is_cuda) or t.dtype != torch.int32 or not t.is_contiguous():
            raise ValueError("%s must be a contiguous int32 device tensor" % name)
    rows = rowPtr.numel() - 1
    dc = torch.empty(cols, dtype=torch.int32, device=rowPtr.device)
    dr = torch.empty(rows, dtype=torch.int32, device=rowPtr.device)
    out = (C.c_int * 4)()
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    check(_lib.load().mx_select_device(rows, cols, colInd.numel(), rowPtr.data_ptr(), colInd.data_ptr(), tau_c, tau_r,
                                       dc.data_ptr(), dr.data_ptr(), C.cast(out, C.c_void_p), s))
    return dc, dr, dict(zip(("dCols", "nnzColD", "dRows", "nnzRowD"), out))


def split_device(rowPtr, colInd, val, cols, sel, descColId, descRowId, stream=None):
    """A_dd and the residual A_CD from the selections of select_device(), all device tensors:
    returns (ddRowPtr, ddColInd, ddVal, cdRowPtr, cdColInd, cdVal)."""
    import torch
    rows, nnz = rowPtr.numel() - 1, colInd.numel()
    dt = MX_F64 if val.dtype == torch.float64 else MX_F16
    dev, i32 = rowPtr.device, torch.int32
    nDD = sel["nnzRowD"]
    out = (torch.empty(sel["dRows"] + 1, dtype=i32, device=dev), torch.empty(nDD, dtype=i32, device=dev),
           torch.empty(nDD, dtype=val.dtype, device=dev), torch.empty(rows + 1, dtype=i32, device=dev),
           torch.empty(nnz - nDD, dtype=i32, device=dev), torch.empty(nnz - nDD, dtype=val.dtype, device=dev))
    csel = (C.c_int * 4)(sel["dCols"], sel["nnzColD"], sel["dRows"], sel["nnzRowD"])
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    check(_lib.load().mx_split_device(dt, rows, cols, nnz, rowPtr.data_ptr(), colInd.data_ptr(), val.data_ptr(),
                                      C.cast(csel, C.c_void_p), descColId.data_ptr(), descRowId.data_ptr(),
                                      *[t.data_ptr() for t in out], s))
    return out


def tiles_device(ddRowPtr, ddColInd, ddVal, dCols, stream=None):
    """The tile arrays of A_dd (device tensors as split_device() returns them), built on the device;
    returned as a dict of device tensors (copies; the library's block is released before returning)."""
    import torch
    dt = MX_F64 if ddVal.dtype == torch.float64 else MX_F16
    t = _lib.DeviceTiles()
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    lib = _lib.load()
    check(lib.mx_tiles_device(dt, ddRowPtr.numel() - 1, dCols, ddColInd.numel(), ddRowPtr.data_ptr(), ddColInd.data_ptr(),
                              ddVal.data_ptr(), C.byref(t), s))
    try:
        def take(ptr, n, dtype):
            out = torch.empty(n, dtype=dtype, device=ddRowPtr.device)
            if n:
                hip = C.CDLL("libamdhip64.so")
                hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
                if hip.hipMemcpy(out.data_ptr(), ptr, n * out.element_size(), 3) != 0:  # device to device
                    raise MxError("hipMemcpy failed")
            return out
        bit_t = torch.int32 if dt == MX_F64 else torch.int64
        return {"chunkNum": t.chunkNum, "totalTcFrags": t.totalTcFrags, "fragK": t.fragK, "tcValCount": t.tcValCount,
                "chunkPtr": take(t.chunkPtr, t.chunkNum + 1, torch.int32),
                "sparse_AToX_index": take(t.sparse_AToX_index, t.totalTcFrags * t.fragK, torch.int32),
                "fragPtr": take(t.fragPtr, t.totalTcFrags + 1, torch.int32),
                "fragBit": take(t.fragBit, t.totalTcFrags, bit_t),
                "tcVal": take(t.tcVal, t.tcValCount, ddVal.dtype)}
    finally:
        lib.mx_tiles_device_free(C.byref(t))


class Partition:
    """Result of the cascaded extraction (column pass tau_c, then row pass tau_r)."""

    ARRAYS = ("descColId", "newArray", "rId", "newArray_", "ddRowPtr", "ddColInd", "ddVal", "chunkPtr",
              "sparse_AToX_index", "fragPtr", "fragBit", "tcVal", "cdRowPtr", "cdColInd", "cdVal")

    def __init__(self, A, tau_c, tau_r, device=False):
        """device=True: the extraction runs on the GPU (mx_partition_create_device); same result.  device=None:
        what the reference's surface does (matxtract_preprocess, the CLI): the GPU for a matrix of two million
        entries or more when there is one, the host otherwise."""
        self._h = C.c_void_p()
        self._A = A  # keep the input arrays alive during the call
        st = A.struct()
        if device is None:
            device = A.nnz >= (1 << 21) and (tau_c != 0 or tau_r != 0) and _lib.load().mx_device_count() > 0
        create = _lib.load().mx_partition_create_device if device else _lib.load().mx_partition_create
        check(create(C.byref(st), float(tau_c), float(tau_r), C.byref(self._h)))
        self._bind()

    @classmethod
    def load(cls, path, dtype=MX_F64):
        """A partition written by save() (mx_partition_load)."""
        self = cls.__new__(cls)
        self._h = C.c_void_p()
        self._A = None
        check(_lib.load().mx_partition_load(os.fsencode(path), int(dtype), C.byref(self._h)))
        self._bind()
        return self

    def save(self, path):
        """Write the partition to `path`: the reference's _preprocessed.dat fields, then the rest."""
        check(_lib.load().mx_partition_save(self._h, os.fsencode(path)))

    def _bind(self):
        """The counts now; the arrays when one of them is asked for (a partition made on the device keeps them
        there until then, and a plan made from it never asks)."""
        v = _lib.PartitionView()
        check(_lib.load().mx_partition_counts(self._h, C.byref(v)))
        for name, _ in _lib.PartitionView._fields_:
            if name not in self.ARRAYS:
                setattr(self, name, getattr(v, name))
        self.tau_c, self.tau_r = float(v.tau_c), float(v.tau_r)

    def __getattr__(self, name):
        if name not in Partition.ARRAYS or "_h" not in self.__dict__:
            raise AttributeError(name)
        v = _lib.PartitionView()
        check(_lib.load().mx_partition_get(self._h, C.byref(v)))
        vt = _np_dtype(v.dtype)
        bt = np.uint32 if v.dtype == MX_F64 else np.uint64
        self.descColId = _view(v.descColId, v.cols if v.descColId else 0, np.int32)
        self.newArray = _view(v.newArray, v.sCols, np.int32)
        self.rId = _view(v.rId, v.dRows, np.int32)
        self.newArray_ = _view(v.newArray_, v.sRows, np.int32)
        self.ddRowPtr = _view(v.ddRowPtr, v.dRows + 1, np.int32)
        self.ddColInd = _view(v.ddColInd, v.nnzRowD, np.int32)
        self.ddVal = _view(v.ddVal, v.nnzRowD, vt)
        self.chunkPtr = _view(v.chunkPtr, v.chunkNum + 1, np.int32)
        self.sparse_AToX_index = _view(v.sparse_AToX_index, v.totalTcFrags * v.fragK, np.int32)
        self.fragPtr = _view(v.fragPtr, v.totalTcFrags + 1, np.int32)
        self.fragBit = _view(v.fragBit, v.totalTcFrags, bt)
        self.tcVal = _view(v.tcVal, v.tcValCount, vt)
        self.cdRowPtr = _view(v.cdRowPtr, v.rows + 1, np.int32)
        self.cdColInd = _view(v.cdColInd, v.nnzCD, np.int32)
        self.cdVal = _view(v.cdVal, v.nnzCD, vt)
        return self.__dict__[name]

    @property
    def hash(self):
        return _lib.load().mx_partition_hash(self._h)

    def close(self):
        if self._h:
            _lib.load().mx_partition_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def debug_fused_misplaced(on):
    """Sets (or clears) the word a misplaced workgroup of a one-launch product sets (mx_debug_fused_misplaced)."""
    check(_lib.load().mx_debug_fused_misplaced(1 if on else 0))


def time_rotate(plans, xs, ys, warm=200, iters=4000):
    """Mean ms per product of a train that takes the plans in turn (mx_time_rotate); xs, ys: one device
    tensor per plan."""
    n = len(plans)
    assert n >= 1 and len(xs) == n and len(ys) == n
    for p, x, y in zip(plans, xs, ys):
        p._check_vec(x, p.cols, "x")
        p._check_vec(y, p.rows, "y")
    hp = (C.c_void_p * n)(*[p._h.value for p in plans])
    xp = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
    yp = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
    ms = C.c_double()
    check(_lib.load().mx_time_rotate(hp, xp, yp, n, int(warm), int(iters), C.byref(ms)))
    return ms.value


def slice_layout(A, nCU=256, sel=None, device=False, fused=False):
    """The layout of the column-slice kernel for matrix A as a dict of numpy arrays and sizes (see
    mx_slice_layout in include/matxtract_hip.h), built on the host, or with device=True on the GPU
    (mx_slice_layout_device: the same arrays).  `sel`: optional mask of the rows to include (host
    route only).  fused=True: the layout of the one-launch form (mx_slice_layout_fused; out["fused"]
    tells whether the matrix suited it)."""
    v = _lib.SliceLayoutView()
    st = A.struct()
    selp = None
    if sel is not None:
        sel = np.ascontiguousarray(sel, dtype=np.uint8)
        assert sel.shape == (A.rows,) and not device
        selp = sel.ctypes.data
    if fused:
        assert sel is None and not device
        check(_lib.load().mx_slice_layout_fused(C.byref(st), int(nCU), C.byref(v)))
    elif device:
        check(_lib.load().mx_slice_layout_device(C.byref(st), int(nCU), C.byref(v)))
    else:
        check(_lib.load().mx_slice_layout(C.byref(st), int(nCU), selp, C.byref(v)))
    try:
        out = {n: int(getattr(v, n)) for n in ("nWG", "S", "sliceCols", "waves", "stepEntries", "batchEntries", "cap",
                                               "chunks", "batches", "vrows", "nLight", "nHeavy", "lightSegs")}
        vt = _np_dtype(A.dtype)
        out["wgDesc"] = _view(v.wgDesc, v.nWG * 4, np.int32).reshape(-1, 4).copy()
        out["waveDesc"] = _view(v.waveDesc, v.nWG * v.waves * 4, np.int32).reshape(-1, 4).copy()
        out["chunkEnd"] = _view(v.chunkEnd, v.chunks, np.int32).copy()
        out["segPtr"] = _view(v.segPtr, A.rows + 1, np.int32).copy()
        out["segIdx"] = _view(v.segIdx, v.vrows, np.int32).copy()
        out["rowInfo"] = _view(v.rowInfo, A.rows, np.int32).copy()
        out["lightInfo"] = _view(v.lightInfo, v.nLight * 4, np.int32).reshape(-1, 4).copy()
        out["heavyInfo"] = _view(v.heavyInfo, v.nHeavy * 4, np.int32).reshape(-1, 4).copy()
        out["ecol"] = _view(v.ecol, v.nEcol, np.uint16).copy()
        out["eval"] = _view(v.eval, v.nEcol, vt).copy()
        out["nDict"] = int(v.nDict)
        out["ecode"] = _view(v.ecode, v.nEcol if v.nDict else 0, np.uint8).copy()
        out["dict"] = _view(v.dict, 256 if v.nDict else 0, vt).copy()
        out["fused"] = int(v.fused)
        if v.fused:
            for n in ("groupRows", "nGroups", "placesPerRow"):
                out[n] = int(getattr(v, n))
            out["wgGroups"] = _view(v.wgGroups, v.nWG * 2, np.int32).reshape(-1, 2).copy()
            out["groupNeed"] = _view(v.groupNeed, v.nGroups, np.int32).copy()
            out["fusedTarget"] = _view(v.fusedTarget, v.chunks * 64, np.int32).copy()
            out["rowVrows"] = _view(v.rowVrows, v.nGroups * v.groupRows, np.uint8).copy()
    finally:
        _lib.load().mx_slice_layout_free(C.byref(v))
    return out


def plan_layout(part, flags=MX_PLAN_DEFAULT, nCU=256):
    """The host half of a plan for partition `part` (no GPU needed): the CSR part in the caller's
    numbering and the two tile layouts as the kernels read them, as a dict of numpy arrays (see
    mx_plan_layout in include/matxtract_hip.h)."""
    v = _lib.PlanLayoutView()
    check(_lib.load().mx_plan_layout(part._h, int(flags), int(nCU), C.byref(v)))
    try:
        vt = _np_dtype(part.dtype)
        out = {n: int(getattr(v, n)) for n in ("rows", "cols", "csr_nnz", "fragM", "fragK", "slots", "csr_variant")}
        out["est_rows_us"], out["est_slices_us"] = float(v.est_rows_us), float(v.est_slices_us)
        out["csrRowPtr"] = _view(v.csrRowPtr, v.rows + 1, np.int32).copy()
        out["csrColInd"] = _view(v.csrColInd, v.csr_nnz, np.int32).copy()
        out["csrVal"] = _view(v.csrVal, v.csr_nnz, vt).copy()
        out["stripRows"] = _view(v.stripRows, v.rows, np.uint8).copy()
        out["tiles"] = []
        for t in v.tiles:
            out["tiles"].append({
                "steps": int(t.steps), "nWaves": int(t.nWaves), "chunks": int(t.chunks), "nnz": int(t.nnz),
                "dense": bool(t.dense),
                "hdr": _view(t.hdr, t.steps * 32, np.int32).reshape(-1, 32).copy(),
                "atox": _view(t.atox, t.steps * 64, np.int32).reshape(-1, 64).copy(),
                "waveDesc": _view(t.waveDesc, t.nWaves * 8, np.int32).reshape(-1, 8).copy(),
                "valOffset": _view(t.valOffset, t.steps, np.int32).copy(),
                "val": _view(t.val, t.nVal, vt).copy(),
            })
    finally:
        _lib.load().mx_plan_layout_free(C.byref(v))
    return out


def tile_steps(chunk_blocks, slots, block_values, per_min, nCU):
    """The steps and waves of a tile layout from the block counts of its chunks (mx_tile_steps, no GPU
    needed): dict with stepDesc [steps, 10], chunkBlock0, waveDesc [nWaves, 8], totalBlocks."""
    cb = np.ascontiguousarray(chunk_blocks, dtype=np.int32)
    v = _lib.TileStepsView()
    check(_lib.load().mx_tile_steps(_p(cb), cb.size, int(slots), int(block_values), int(per_min), int(nCU), C.byref(v)))
    try:
        return {"steps": int(v.steps), "nWaves": int(v.nWaves), "totalBlocks": int(v.totalBlocks),
                "stepDesc": _view(v.stepDesc, v.steps * 10, np.int32).reshape(-1, 10).copy(),
                "chunkBlock0": _view(v.chunkBlock0, cb.size, np.int32).copy(),
                "waveDesc": _view(v.waveDesc, v.nWaves * 8, np.int32).reshape(-1, 8).copy()}
    finally:
        _lib.load().mx_tile_steps_free(C.byref(v))


def tune_tau(A, levels=5, flags=MX_PLAN_DEFAULT, warm=20, iters=200):
    """(tau_c, tau_r, table) for matrix A on this device: every grid point with tau_c >= tau_r is
    partitioned, planned and timed (mx_tune_tau); table = [(tau_c, tau_r, ms, tile_nnz), ...]."""
    st = A.struct()
    cap = levels * (levels + 1) // 2
    table = (_lib.TauPoint * cap)()
    c, r, n = C.c_float(), C.c_float(), C.c_int()
    check(_lib.load().mx_tune_tau(C.byref(st), int(levels), int(flags), int(warm), int(iters), C.byref(c), C.byref(r),
                                  table, cap, C.byref(n)))
    return c.value, r.value, [(t.tau_c, t.tau_r, t.ms_total, t.tile_nnz) for t in table[:n.value]]


def estimate_tau(A, levels=5):
    """(tau_c, tau_r, table) for matrix A from counts alone (mx_estimate_tau): nothing is planned or
    timed; table = [(tau_c, tau_r, saved_us, tile_entries), ...]."""
    st = A.struct()
    cap = levels * (levels + 1) // 2
    table = (_lib.TauEstimate * cap)()
    c, r, n = C.c_float(), C.c_float(), C.c_int()
    check(_lib.load().mx_estimate_tau(C.byref(st), int(levels), C.byref(c), C.byref(r), table, cap, C.byref(n)))
    return c.value, r.value, [(t.tau_c, t.tau_r, t.saved_us, t.tile_entries) for t in table[:n.value]]


def _torch_dtype(dt):
    import torch
    return torch.float64 if dt == MX_F64 else torch.float16


class Plan:
    """A partition resident on the GPU; ``spmv`` computes y = A x there."""

    def __init__(self, partition, flags=MX_PLAN_DEFAULT):
        self._h = C.c_void_p()
        check(_lib.load().mx_plan_create(partition._h, int(flags), C.byref(self._h)))
        info = _lib.PlanInfo()
        check(_lib.load().mx_plan_get_info(self._h, C.byref(info)))
        self.info = {k: getattr(info, k) for k, _ in _lib.PlanInfo._fields_}
        self.dtype, self.rows, self.cols, self.nnz = info.dtype, info.rows, info.cols, info.nnz

    @classmethod
    def from_device_csr(cls, rowPtr, colInd, val, cols, flags=MX_PLAN_DEFAULT):
        """A plan from a CSR matrix held in torch device tensors (int32 rowPtr and colInd, float64 or
        float16 val): mx_plan_create_device_csr; the matrix never crosses to the host."""
        import torch
        for name, t in (("rowPtr", rowPtr), ("colInd", colInd)):
            if (not t.is_cuda) or t.dtype != torch.int32 or not t.is_contiguous():
                raise ValueError("%s must be a contiguous int32 device tensor" % name)
        if (not val.is_cuda) or val.dtype not in (torch.float64, torch.float16) or not val.is_contiguous() \
                or val.numel() != colInd.numel():
            raise ValueError("val must be a contiguous float64 or float16 device tensor as long as colInd")
        self = cls.__new__(cls)
        self._h = C.c_void_p()
        dt = MX_F64 if val.dtype == torch.float64 else MX_F16
        check(_lib.load().mx_plan_create_device_csr(dt, rowPtr.numel() - 1, int(cols), colInd.numel(), rowPtr.data_ptr(),
                                                    colInd.data_ptr(), val.data_ptr(), int(flags), C.byref(self._h)))
        info = _lib.PlanInfo()
        check(_lib.load().mx_plan_get_info(self._h, C.byref(info)))
        self.info = {k: getattr(info, k) for k, _ in _lib.PlanInfo._fields_}
        self.dtype, self.rows, self.cols, self.nnz = info.dtype, info.rows, info.cols, info.nnz
        return self

    @classmethod
    def from_device(cls, rowPtr, colInd, val, cols, tau_c, tau_r, flags=MX_PLAN_DEFAULT):
        """A hybrid plan from a CSR matrix held in torch device tensors and the two extraction
        fractions: mx_plan_create_device -- extraction, decisions and layouts on the device."""
        import torch
        for name, t in (("rowPtr", rowPtr), ("colInd", colInd)):
            if (not t.is_cuda) or t.dtype != torch.int32 or not t.is_contiguous():
                raise ValueError("%s must be a contiguous int32 device tensor" % name)
        if (not val.is_cuda) or val.dtype not in (torch.float64, torch.float16) or not val.is_contiguous() \
                or val.numel() != colInd.numel():
            raise ValueError("val must be a contiguous float64 or float16 device tensor as long as colInd")
        self = cls.__new__(cls)
        self._h = C.c_void_p()
        dt = MX_F64 if val.dtype == torch.float64 else MX_F16
        check(_lib.load().mx_plan_create_device(dt, rowPtr.numel() - 1, int(cols), colInd.numel(), rowPtr.data_ptr(),
                                                colInd.data_ptr(), val.data_ptr(), float(tau_c), float(tau_r), int(flags),
                                                C.byref(self._h)))
        info = _lib.PlanInfo()
        check(_lib.load().mx_plan_get_info(self._h, C.byref(info)))
        self.info = {k: getattr(info, k) for k, _ in _lib.PlanInfo._fields_}
        self.dtype, self.rows, self.cols, self.nnz = info.dtype, info.rows, info.cols, info.nnz
        return self

    def arrays(self):
        """{name: bytes} of every device array of the plan (mx_plan_arrays), for tests that compare
        two routes of making a plan."""
        cap = 48
        buf = (_lib.PlanArray * cap)()
        n = C.c_int(0)
        check(_lib.load().mx_plan_arrays(self._h, buf, cap, C.byref(n)))
        try:
            return {buf[i].name.decode(): C.string_at(buf[i].data, buf[i].bytes) for i in range(n.value)}
        finally:
            _lib.load().mx_plan_arrays_free(buf, n.value)

    def _check_vec(self, t, n, name):
        if (not t.is_cuda) or t.dtype != _torch_dtype(self.dtype) or t.numel() != n or not t.is_contiguous():
            raise ValueError("%s must be a contiguous device tensor of %d %s" % (name, n, _torch_dtype(self.dtype)))

    def spmv(self, x, y=None, stream=None):
        """y = A x; x, y torch device tensors.  Launches on `stream` (default: torch's current)."""
        import torch
        if y is None:
            y = torch.empty(self.rows, dtype=x.dtype, device=x.device)
        self._check_vec(x, self.cols, "x")
        self._check_vec(y, self.rows, "y")
        s = torch.cuda.current_stream().cuda_stream if stream is None else stream
        check(_lib.load().mx_spmv(self._h, x.data_ptr(), y.data_ptr(), s))
        return y

    def spmv_static(self, x, y, stream=None):
        """y = A x without any allocation: the kernels' partial sums go to the library's fixed
        device array (mx_spmv_static).  y must be given."""
        import torch
        self._check_vec(x, self.cols, "x")
        self._check_vec(y, self.rows, "y")
        s = torch.cuda.current_stream().cuda_stream if stream is None else stream
        check(_lib.load().mx_spmv_static(self._h, x.data_ptr(), y.data_ptr(), s))
        return y

    def spmv_repeat(self, x, y, n, stream=None):
        """n back-to-back y = A x, queued from C (no Python between launches)."""
        import torch
        self._check_vec(x, self.cols, "x")
        self._check_vec(y, self.rows, "y")
        s = torch.cuda.current_stream().cuda_stream if stream is None else stream
        check(_lib.load().mx_spmv_repeat(self._h, x.data_ptr(), y.data_ptr(), int(n), s))
        return y

    def spmv_host(self, x):
        x = np.ascontiguousarray(x, dtype=_np_dtype(self.dtype))
        if x.size != self.cols:
            raise ValueError("x must have %d entries" % self.cols)
        y = np.zeros(self.rows, x.dtype)
        check(_lib.load().mx_spmv_host(self._h, _p(x), _p(y)))
        return y

    def time(self, x, y, warm=200, iters=4000, parts=True):
        """Mean ms per SpMV by HIP events on the plan's stream -> (total, tile, csr)."""
        self._check_vec(x, self.cols, "x")
        self._check_vec(y, self.rows, "y")
        t, tt, tc = C.c_double(), C.c_double(), C.c_double()
        check(_lib.load().mx_time(self._h, x.data_ptr(), y.data_ptr(), warm, iters, C.byref(t),
                                  C.byref(tt) if parts else None, C.byref(tc) if parts else None))
        return t.value, tt.value, tc.value

    def time_kernels(self, x, y, warm=200, iters=4000):
        """Every kernel launch of one product timed alone (mx_time_kernels) ->
        [{"name", "ms", "algorithmic_bytes", "nnz"}, ...] in launch order."""
        self._check_vec(x, self.cols, "x")
        self._check_vec(y, self.rows, "y")
        recs = (_lib.KernelTime * 8)()
        n = C.c_int()
        check(_lib.load().mx_time_kernels(self._h, x.data_ptr(), y.data_ptr(), warm, iters, recs, 8, C.byref(n)))
        return [{"name": r.name.decode(), "ms": r.ms, "algorithmic_bytes": r.algorithmic_bytes, "nnz": r.nnz}
                for r in recs[:n.value]]

    def time_csr_main(self, x, y, warm=200, iters=4000):
        """Mean ms per launch of the CSR part's main kernel alone."""
        self._check_vec(x, self.cols, "x")
        self._check_vec(y, self.rows, "y")
        t = C.c_double()
        check(_lib.load().mx_time_csr_main(self._h, x.data_ptr(), y.data_ptr(), warm, iters, C.byref(t)))
        return t.value

    def close(self):
        if self._h:
            _lib.load().mx_plan_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def cdspmv(A, x, y, warm=0, iters=0):
    """Reference cdspmv(): y += A x, host arrays in and out -> (y, cdTime_ms, cdPre_ms)."""
    vt = _np_dtype(A.dtype)
    x = np.ascontiguousarray(x, dtype=vt)
    y = np.array(y, dtype=vt)
    t, pre = C.c_double(), C.c_double()
    fn = _lib.load().mx_cdspmv_f64 if A.dtype == MX_F64 else _lib.load().mx_cdspmv_f16
    check(fn(_p(A.val), _p(A.rowPtr), _p(A.colInd), _p(x), _p(y), A.rows, A.cols, A.nnz, warm, iters,
             C.byref(t), C.byref(pre)))
    return y, t.value, pre.value


def du_tcspmv(part, x_d, y_d=None, warm=0, iters=0):
    """Reference du_tcspmv_fp64 / du_tcspmv_fp16_v2 on a partition's canonical tile arrays."""
    dt = part.dtype
    vt = _np_dtype(dt)
    x_d = np.ascontiguousarray(x_d, dtype=vt)
    y = np.zeros(part.dRows, vt) if y_d is None else np.array(y_d, dtype=vt)
    t = C.c_double()
    fn = _lib.load().mx_du_tcspmv_f64 if dt == MX_F64 else _lib.load().mx_du_tcspmv_f16
    check(fn(_p(part.chunkPtr), _p(part.fragPtr), _p(part.fragBit), _p(part.tcVal), _p(part.sparse_AToX_index),
             _p(x_d), _p(y), part.dRows, part.dCols, warm, iters, C.byref(t)))
    return y, t.value
