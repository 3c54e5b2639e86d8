"""ctypes binding of the CPU oracle (oracle/oracle.c).  TEST INFRASTRUCTURE ONLY.

Imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py as the checker.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
IDX_MAX = 0xFFFFFFFF
ROW_WINDOW = 8


def build(force=False):
    """Compile oracle.c with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Csr(C.Structure):
    _fields_ = [("rows", C.c_uint32), ("cols", C.c_uint32), ("nnzs", C.c_uint32),
                ("declared_nnz", C.c_uint32),
                ("row_ptr", C.POINTER(C.c_uint32)), ("col_idx", C.POINTER(C.c_uint32)),
                ("values", C.c_void_p), ("status", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        L.orc_mtx_read.restype = C.POINTER(_Csr)
        L.orc_mtx_read.argtypes = [C.c_char_p, C.c_int]
        L.orc_csr_free.argtypes = [C.POINTER(_Csr)]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_verdict_rel.restype = C.c_size_t
        L.orc_verdict_rel_abs.restype = C.c_size_t
        L.orc_max_threads.restype = C.c_int
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_f16_array(_p(x), _p(out), C.c_size_t(x.size))
    return out


def f16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_f16_to_f32_array(_p(h), _p(out), C.c_size_t(h.size))
    return out


def f32_to_bf16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_bf16_array(_p(x), _p(out), C.c_size_t(x.size))
    return out


def bf16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_bf16_to_f32_array(_p(h), _p(out), C.c_size_t(h.size))
    return out


def mtx_read(path, dtype):
    """dtype 'fp16' / 'bf16' -> values as uint16 bit patterns; 'tf32' -> float32.
    Returns dict(rows, cols, nnzs, declared_nnz, row_ptr, col_idx, values) or
    raises OSError / ValueError following the oracle's status code."""
    es = 4 if dtype == "tf32" else 2
    m = lib().orc_mtx_read(os.fsencode(path), {"fp16": 2, "bf16": 3, "tf32": 4}[dtype])
    try:
        s = m.contents
        if s.status == 1:
            raise OSError("cannot open %s" % path)
        if s.status == 2:
            raise ValueError("cannot parse the size line of %s" % path)
        if s.status == 4:
            raise ValueError("index out of range in %s" % path)
        if s.status != 0:
            raise MemoryError()
        n = s.nnzs
        row_ptr = np.ctypeslib.as_array(s.row_ptr, (s.rows + 1,)).copy()
        col_idx = np.ctypeslib.as_array(s.col_idx, (max(n, 1),))[:n].copy()
        vt = np.uint16 if es == 2 else np.float32
        vals = np.ctypeslib.as_array(C.cast(s.values, C.POINTER(np.ctypeslib.as_ctypes_type(vt))),
                                     (max(n, 1),))[:n].copy()
        return dict(rows=s.rows, cols=s.cols, nnzs=n, declared_nnz=s.declared_nnz,
                    row_ptr=row_ptr, col_idx=col_idx, values=vals)
    finally:
        lib().orc_csr_free(m)


def csr_validate(rows, cols, row_ptr, col_idx):
    row_ptr = _c(row_ptr, np.uint32)
    col_idx = _c(col_idx, np.uint32)
    return lib().orc_csr_validate(C.c_uint32(rows), C.c_uint32(cols), C.c_uint32(col_idx.size),
                                  _p(row_ptr), _p(col_idx))


def csr_to_btcf(rows, cols, row_ptr, col_idx, values, dtype, transpose=False, cw=None):
    """CSR -> condensed tiles (no bitmap).  values: uint16 bits (fp16) or float32 (tf32)."""
    es = 4 if dtype == "tf32" else 2
    if cw is None:
        cw = 8 if dtype == "tf32" else 16
    vt = np.uint16 if es == 2 else np.float32
    row_ptr = _c(row_ptr, np.uint32)
    col_idx = _c(col_idx, np.uint32)
    values = _c(values, vt)
    W = C.c_uint32()
    T = C.c_uint32()
    lib().orc_btcf_count(C.c_uint32(rows), _p(row_ptr), _p(col_idx), C.c_uint32(cw),
                         C.byref(W), C.byref(T))
    W, T = W.value, T.value
    rowOffset = np.zeros(W + 1, np.uint32)
    tcA2B = np.empty(T * cw, np.uint32)
    data = np.zeros(T * ROW_WINDOW * cw, vt)
    rowIdx = np.empty(W, np.uint32)
    lib().orc_btcf_fill(C.c_uint32(rows), _p(row_ptr), _p(col_idx), _p(values), C.c_uint32(es),
                        C.c_uint32(cw), C.c_int(int(transpose)),
                        _p(rowOffset), _p(tcA2B), _p(data), _p(rowIdx))
    return dict(rows=rows, cols=cols, nnzs=int(col_idx.size), dtype=dtype, cw=cw,
                total_row_windows=(rows + ROW_WINDOW - 1) // ROW_WINDOW,
                eff_row_windows=W, total_tiles=T,
                rowOffset=rowOffset, tcA2B=tcA2B, data=data, rowIdx=rowIdx)


def csr_to_bitmap(rows, cols, row_ptr, col_idx, values, dtype, transpose=False, as_reference=False):
    """CSR -> bitmap-compressed tiles.  as_reference=True indexes tcBit exactly as
    the reference does (neighbouring 8 x 16 tiles share a word)."""
    es = 4 if dtype == "tf32" else 2
    cw = 8 if dtype == "tf32" else 16
    words = 1 if cw == 8 else 2
    vt = np.uint16 if es == 2 else np.float32
    row_ptr = _c(row_ptr, np.uint32)
    col_idx = _c(col_idx, np.uint32)
    values = _c(values, vt)
    W = C.c_uint32()
    T = C.c_uint32()
    lib().orc_btcf_count(C.c_uint32(rows), _p(row_ptr), _p(col_idx), C.c_uint32(cw), C.byref(W), C.byref(T))
    W, T = W.value, T.value
    nnz = int(row_ptr[rows])
    rowOffset = np.zeros(W + 1, np.uint32)
    nnzOffset = np.zeros(T + 1, np.uint32)
    tcA2B = np.empty(T * cw, np.uint32)
    tcBit = np.zeros(T * words, np.uint64)
    data = np.zeros(nnz, vt)
    rowIdx = np.empty(W, np.uint32)
    lib().orc_bitmap_fill(C.c_uint32(rows), _p(row_ptr), _p(col_idx), _p(values), C.c_uint32(es), C.c_uint32(cw),
                          C.c_int(int(transpose)), C.c_int(int(as_reference)),
                          _p(rowOffset), _p(nnzOffset), _p(tcA2B), _p(tcBit), _p(data), _p(rowIdx))
    return dict(rows=rows, cols=cols, nnzs=nnz, dtype=dtype, cw=cw,
                total_row_windows=(rows + ROW_WINDOW - 1) // ROW_WINDOW, eff_row_windows=W, total_tiles=T,
                rowOffset=rowOffset, nnzOffset=nnzOffset, tcA2B=tcA2B, tcBit=tcBit, data=data, rowIdx=rowIdx)


def group(rowOffset, rowIdx, min_len=32):
    """Window list -> groups of at most tgl tiles: (tgl, groupOffset, groupRowIdx, atomic)."""
    rowOffset = _c(rowOffset, np.uint32)
    rowIdx = _c(rowIdx, np.uint32)
    W = rowIdx.size
    tgl = C.c_uint32()
    L = lib()
    L.orc_group.restype = C.c_uint32
    n = L.orc_group(C.c_uint32(W), _p(rowOffset), _p(rowIdx), C.c_uint32(min_len), C.byref(tgl), None, None, None)
    groupOffset = np.zeros(n + 1, np.uint32)
    groupRowIdx = np.zeros(n, np.uint32)
    atomic = np.zeros(n, np.uint8)
    L.orc_group(C.c_uint32(W), _p(rowOffset), _p(rowIdx), C.c_uint32(min_len), C.byref(tgl),
                _p(groupOffset), _p(groupRowIdx), _p(atomic))
    return tgl.value, groupOffset, groupRowIdx, atomic


def spmm_csr_f16(rows, N, row_ptr, col_idx, vals_bits, B_bits, want_absdot=False, threads=0):
    row_ptr = _c(row_ptr, np.uint32)
    col_idx = _c(col_idx, np.uint32)
    vals_bits = _c(vals_bits, np.uint16)
    B_bits = _c(B_bits, np.uint16)
    Cm = np.empty((rows, N), np.uint16)
    mag = np.empty((rows, N), np.float32) if want_absdot else None
    lib().orc_spmm_csr_f16(C.c_uint32(rows), C.c_uint32(N), _p(row_ptr), _p(col_idx), _p(vals_bits),
                           _p(B_bits), _p(Cm), _p(mag) if want_absdot else None, C.c_int(threads))
    return (Cm, mag) if want_absdot else Cm


def spmm_csr_bf16(rows, N, row_ptr, col_idx, vals_bits, B_bits, want_absdot=False, threads=0):
    row_ptr = _c(row_ptr, np.uint32)
    col_idx = _c(col_idx, np.uint32)
    vals_bits = _c(vals_bits, np.uint16)
    B_bits = _c(B_bits, np.uint16)
    Cm = np.empty((rows, N), np.uint16)
    mag = np.empty((rows, N), np.float32) if want_absdot else None
    lib().orc_spmm_csr_bf16(C.c_uint32(rows), C.c_uint32(N), _p(row_ptr), _p(col_idx), _p(vals_bits),
                            _p(B_bits), _p(Cm), _p(mag) if want_absdot else None, C.c_int(threads))
    return (Cm, mag) if want_absdot else Cm


def spmm_csr_f32(rows, N, row_ptr, col_idx, vals, B, want_absdot=False, trunc_tf32=False, threads=0):
    row_ptr = _c(row_ptr, np.uint32)
    col_idx = _c(col_idx, np.uint32)
    vals = _c(vals, np.float32)
    B = _c(B, np.float32)
    Cm = np.empty((rows, N), np.float32)
    mag = np.empty((rows, N), np.float32) if want_absdot else None
    lib().orc_spmm_csr_f32(C.c_uint32(rows), C.c_uint32(N), _p(row_ptr), _p(col_idx), _p(vals), _p(B),
                           _p(Cm), _p(mag) if want_absdot else None, C.c_int(int(trunc_tf32)),
                           C.c_int(threads))
    return (Cm, mag) if want_absdot else Cm


def spmm_btcf(btcf, B, N):
    """Tile-order SpMM on a dict as returned by csr_to_btcf (row-major tiles only)."""
    rows, W = btcf["rows"], btcf["eff_row_windows"]
    if btcf["dtype"] in ("fp16", "bf16"):
        assert btcf["cw"] == 16
        B = _c(B, np.uint16)
        Cm = np.empty((rows, N), np.uint16)
        fn = lib().orc_spmm_btcf_f16 if btcf["dtype"] == "fp16" else lib().orc_spmm_btcf_bf16
        fn(C.c_uint32(rows), C.c_uint32(N), C.c_uint32(W), _p(btcf["rowOffset"]),
                                _p(btcf["tcA2B"]), _p(btcf["data"]), _p(btcf["rowIdx"]), _p(B), _p(Cm))
    else:
        B = _c(B, np.float32)
        Cm = np.empty((rows, N), np.float32)
        lib().orc_spmm_btcf_f32(C.c_uint32(rows), C.c_uint32(N), C.c_uint32(W), C.c_uint32(btcf["cw"]),
                                _p(btcf["rowOffset"]), _p(btcf["tcA2B"]), _p(btcf["data"]),
                                _p(btcf["rowIdx"]), _p(B), _p(Cm))
    return Cm


def tile_mma_f16(A_bits, B_bits, M, N, K):
    A_bits = _c(A_bits, np.uint16)
    B_bits = _c(B_bits, np.uint16)
    out = np.empty((M, N), np.float32)
    lib().orc_tile_mma_f16(_p(A_bits), _p(B_bits), _p(out), M, N, K)
    return out


def tile_mma_f32(A, B, M, N, K):
    A = _c(A, np.float32)
    B = _c(B, np.float32)
    out = np.empty((M, N), np.float32)
    lib().orc_tile_mma_f32(_p(A), _p(B), _p(out), M, N, K)
    return out


def tile_accum_f32(A, B, M, N, K, T):
    A = _c(A, np.float32)
    B = _c(B, np.float32)
    out = np.empty((M, N), np.float32)
    lib().orc_tile_accum_f32(_p(A), _p(B), _p(out), M, N, K, T)
    return out


def verdict_rel(expected, actual, tol=1e-2):
    e = _c(expected, np.float32).ravel()
    a = _c(actual, np.float32).ravel()
    return lib().orc_verdict_rel(_p(e), _p(a), C.c_size_t(e.size), C.c_float(tol))


def verdict_rel_abs(actual, ref, tol=1e-2):
    a = _c(actual, np.float32).ravel()
    r = _c(ref, np.float32).ravel()
    return lib().orc_verdict_rel_abs(_p(a), _p(r), C.c_size_t(a.size), C.c_double(tol))


def max_threads():
    return lib().orc_max_threads()
