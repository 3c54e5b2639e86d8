"""ctypes binding of libhspmm.so (include/hspmm.h).

Every function here calls the C ABI; there is no Python or CPU fallback for the
device operator: if the library is missing, or no gfx950 device is present,
`Plan` raises.
"""
import ctypes as C
import os
import subprocess

import numpy as np

FP16 = 0            # HSPMM_FP16, reference -DUSE_FP16 (src/common.h:14-19)
TF32 = 1            # HSPMM_TF32, reference -DUSE_TF32 (src/common.h:26-43), fp32 storage
BF16 = 2            # HSPMM_BF16, reference -DUSE_BF16 (src/common.h:20-25)
IDX_MAX = 0xFFFFFFFF
ROW_WINDOW = 8

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libhspmm.so")
_lib = None


class HspmmError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("hspmm error %d: %s" % (code, text))
        self.code = code


def library_path():
    return _LIB


def build_library(force=True, experimental=False):
    """Compile the HIP sources for gfx950 (hipcc cross-compiles without a GPU).  experimental: also the kernel
    variants that no automatic plan selects (EXPERIMENTAL=1 of csrc/Makefile)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    if experimental:
        cmd.append("EXPERIMENTAL=1")
    if force:
        cmd.insert(1, "-B")
    subprocess.check_call(cmd, stdout=subprocess.DEVNULL)
    # the command-line drivers (fp16_test / tf32_test) link against the library
    # (not with -B: it would also remake their prerequisite, the library, once per driver)
    cli = ["make", "-C", os.path.join(_HERE, "host")]
    if force:
        subprocess.check_call(cli + ["clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(cli + ["-j4", "fp16_test", "bf16_test", "tf32_test", "fp16_transposed_test", "tf32_k4_test"],
                          stdout=subprocess.DEVNULL)
    return _LIB


def cli_path(name):
    """Path of a built command-line driver: 'fp16_test', 'bf16_test', 'tf32_test', or
    'fp16_transposed_test' (fp16_test built with -DSPARSE_A_TRANSPOSE), 'tf32_k4_test' (tf32_test built with
    -DMMA_M16N8K4: 8 x 4 tiles)."""
    return os.path.join(_HERE, "host", name)


class _Csr(C.Structure):
    _fields_ = [("rows", C.c_uint32), ("cols", C.c_uint32), ("nnzs", C.c_uint32),
                ("row_ptr", C.POINTER(C.c_uint32)), ("col_idx", C.POINTER(C.c_uint32)),
                ("values", C.c_void_p)]


class PlanInfo(C.Structure):
    _fields_ = [("rows", C.c_uint32), ("cols", C.c_uint32), ("eff_row_windows", C.c_uint32),
                ("total_tiles", C.c_uint32), ("dtype", C.c_int32), ("n_ranges", C.c_uint32),
                ("n_split_windows", C.c_uint32), ("n_partial_slots", C.c_uint32),
                ("compute_units", C.c_uint32), ("n_units", C.c_uint32), ("n_paired_units", C.c_uint32),
                ("device_bytes", C.c_uint64), ("n_panels", C.c_uint32), ("n_panel_steps", C.c_uint32),
                ("n_panel_units", C.c_uint32), ("n_panel_paired_units", C.c_uint32),
                ("n_panel_wide_units", C.c_uint32), ("last_kernel_family", C.c_uint32),
                ("gather_bitmap", C.c_uint32), ("bitmap_from_caller", C.c_uint32), ("panel_stream_mode", C.c_uint32),
                ("group_cuts_kept", C.c_uint32), ("last_mfma_kind", C.c_uint32), ("last_mfma_flops", C.c_uint32),
                ("last_mfma_instructions", C.c_uint64)]


def load_library():
    """Load libhspmm.so; build it first only if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        build_library(force=False)
    # A process that also uses PyTorch must end up with one HIP runtime.  PyTorch
    # ships its own libamdhip64 with the same soname as the system one this
    # library is linked against; whichever is loaded first serves both, and
    # PyTorch does not find the device through the system copy.  So let PyTorch
    # load its runtime first when it is installed.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(_LIB)
    u32, vp, i = C.c_uint32, C.c_void_p, C.c_int
    L.hspmm_last_error.restype = C.c_char_p
    L.hspmm_create.argtypes = [C.POINTER(vp), i, u32, u32, u32, u32, vp, vp, vp, vp]
    L.hspmm_btcf_relayout_sizes.argtypes = [i, u32, u32, vp, vp, C.POINTER(u32)]
    L.hspmm_btcf_relayout_fill.argtypes = [i, u32, i, u32, vp, vp, vp, vp, vp, vp]
    L.hspmm_partition_as_groups.argtypes = [vp, u32, C.POINTER(u32), vp, vp, vp]
    L.hspmm_create_layout.argtypes = [C.POINTER(vp), i, u32, i, u32, u32, u32, u32, vp, vp, vp, vp]
    L.hspmm_run.argtypes = [vp, vp, vp, u32, vp]
    L.hspmm_run_static.argtypes = [vp, vp, vp, u32, vp]
    L.hspmm_prepare.argtypes = [vp, u32]
    L.hspmm_bench.argtypes = [vp, vp, vp, u32, i, i, vp, C.POINTER(C.c_float)]
    L.hspmm_profile.argtypes = [vp, vp, vp, u32, i, vp, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.hspmm_measure_gather.argtypes = [vp, vp, u32, i, vp, C.POINTER(C.c_float), C.POINTER(C.c_uint64)]
    L.hspmm_destroy.argtypes = [vp]
    L.hspmm_destroy.restype = None
    L.hspmm_configure.argtypes = [i, i, i, i]
    L.hspmm_get_config.argtypes = [C.POINTER(i)] * 4
    L.hspmm_get_config.restype = None
    L.hspmm_set_kernel_mode.argtypes = [i]
    L.hspmm_set_window_pairing.argtypes = [i]
    L.hspmm_set_panel_stream.argtypes = [i]
    L.hspmm_has_experimental.argtypes = []
    L.hspmm_set_group_cuts.argtypes = [i]
    L.hspmm_get_plan_info.argtypes = [vp, C.POINTER(PlanInfo)]
    L.hspmm_get_partition.argtypes = [vp, vp, u32]
    L.hspmm_partition_preview.argtypes = [u32, vp, u32, vp, u32, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]
    L.hspmm_partition_preview_grouped.argtypes = [u32, vp, u32, u32, vp, u32, C.POINTER(u32), C.POINTER(u32),
                                                  C.POINTER(u32)]
    L.hspmm_partition_preview_aligned.argtypes = [u32, vp, u32, vp, u32, C.POINTER(u32)]
    L.hspmm_partition_preview_group_cuts.argtypes = [u32, vp, u32, u32, vp, vp, u32, C.POINTER(u32), C.POINTER(u32),
                                                     C.POINTER(u32)]
    L.hspmm_panel_units_preview.argtypes = [i, u32, u32, u32, u32, vp, vp, vp, vp, u32, C.POINTER(u32), vp, vp, vp,
                                            C.POINTER(u32), u32, vp, vp]
    L.hspmm_mtx_load.argtypes = [C.c_char_p, i, C.POINTER(_Csr)]
    L.hspmm_csr_free.argtypes = [C.POINTER(_Csr)]
    L.hspmm_csr_free.restype = None
    L.hspmm_btcf_sizes.argtypes = [i, u32, vp, vp, C.POINTER(u32), C.POINTER(u32)]
    L.hspmm_btcf_fill.argtypes = [i, u32, vp, vp, vp, i, vp, vp, vp, vp]
    L.hspmm_btcf_sizes_cw.argtypes = [i, u32, u32, vp, vp, C.POINTER(u32), C.POINTER(u32)]
    L.hspmm_btcf_fill_cw.argtypes = [i, u32, u32, vp, vp, vp, i, vp, vp, vp, vp]
    L.hspmm_bitmap_sizes.argtypes = [i, u32, vp, vp, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]
    L.hspmm_bitmap_fill.argtypes = [i, u32, vp, vp, vp, i, i, vp, vp, vp, vp, vp, vp]
    L.hspmm_bitmap_expand.argtypes = [i, u32, vp, vp, vp, vp]
    L.hspmm_create_bitmap.argtypes = [C.POINTER(vp), i, u32, u32, u32, u32, vp, vp, vp, vp, vp, vp]
    L.hspmm_group_sizes.argtypes = [u32, vp, u32, C.POINTER(u32), C.POINTER(u32)]
    L.hspmm_group_fill.argtypes = [u32, vp, vp, u32, vp, vp, vp]
    L.hspmm_create_grouped.argtypes = [C.POINTER(vp), i, u32, u32, u32, vp, vp, vp, vp, vp, vp, vp]
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise HspmmError(rc, load_library().hspmm_last_error().decode("utf-8", "replace"))


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None and a.size else None


def _copy_out(ptr, count, dt):
    """numpy copy of `count` elements of type dt at the C pointer `ptr`."""
    if count == 0:
        return np.zeros(0, dt)
    addr = C.cast(ptr, C.c_void_p).value
    nbytes = count * np.dtype(dt).itemsize
    return np.frombuffer((C.c_char * nbytes).from_address(addr), dtype=dt).copy()


def _val_dtype(dtype):
    if dtype in (FP16, BF16):
        return np.uint16
    if dtype == TF32:
        return np.float32
    raise ValueError("dtype must be FP16, TF32 or BF16")


def configure(buffer_stage=0, consumer_warp_num=0, producer_warp_group_num=0, sm_num=0):
    """Scheduler::configure of the reference (src/scheduler.h:33-38)."""
    _check(load_library().hspmm_configure(buffer_stage, consumer_warp_num, producer_warp_group_num, sm_num))


def get_config():
    v = [C.c_int() for _ in range(4)]
    load_library().hspmm_get_config(*[C.byref(x) for x in v])
    return tuple(x.value for x in v)


_kernel_mode = 0


def set_kernel_mode(mode):
    """hspmm_set_kernel_mode: 0 automatic, 1 scalar kernel, 2 wide loads, 3 word loads, 4 LDS-staging
    kernels for every matrix, 5 the same with fp32 products for HSPMM_TF32."""
    global _kernel_mode
    _check(load_library().hspmm_set_kernel_mode(mode))
    _kernel_mode = mode


def get_kernel_mode():
    """The mode last set through set_kernel_mode of this module."""
    return _kernel_mode


def set_window_pairing(mode):
    """0 = automatic, 1 = never, 2 = whenever two adjacent windows share a column list."""
    _check(load_library().hspmm_set_window_pairing(mode))


def set_group_cuts(mode):
    """1: plans made from groups (GBTCF_MTX) cut a window only where the caller's groups end; 0 (default): where
    the plan's cost model puts the cuts.  Read by the next plan creation."""
    _check(load_library().hspmm_set_group_cuts(mode))


def has_experimental():
    """True when the library holds the kernel variants no automatic plan selects (built with EXPERIMENTAL=1)."""
    return bool(load_library().hspmm_has_experimental())


def set_panel_stream(mode):
    """0 = uncompressed tiles (default), 1 = two units per consumer wave of the LDS-staging kernels,
    2 = as 1 with the tiles kept on the device without their zeros (bitmap + stored values)."""
    _check(load_library().hspmm_set_panel_stream(mode))


def mtx_load(path, dtype):
    """load_matrix of the reference (src/utils/load.h:152): .mtx -> CSR dict.
    fp16 / bf16 values are returned as uint16 bit patterns."""
    L = load_library()
    m = _Csr()
    _check(L.hspmm_mtx_load(os.fsencode(path), dtype, C.byref(m)))
    try:
        n = m.nnzs
        vt = _val_dtype(dtype)
        row_ptr = _copy_out(m.row_ptr, m.rows + 1, np.uint32)
        col_idx = _copy_out(m.col_idx, n, np.uint32)
        vals = _copy_out(m.values, n, vt)
        return dict(rows=m.rows, cols=m.cols, nnzs=n, row_ptr=row_ptr, col_idx=col_idx, values=vals)
    finally:
        L.hspmm_csr_free(C.byref(m))


def csr_to_btcf(rows, cols, row_ptr, col_idx, values, dtype, transpose=False, cw=None):
    """CSR2BTCFNOBITMAP of the reference (src/utils/convert.h:146): returns the
    BTCF_MTX_NO_BITMAP fields (src/utils/class.h:74-85) as a dict of numpy arrays.  cw: tile width, the
    element type's default or 4 for TF32 (the reference's -DMMA_M16N8K4 build, src/common.h:28-35)."""
    L = load_library()
    vt = _val_dtype(dtype)
    cw = cw or (8 if dtype == TF32 else 16)
    row_ptr = np.ascontiguousarray(row_ptr, np.uint32)
    col_idx = np.ascontiguousarray(col_idx, np.uint32)
    values = np.ascontiguousarray(values, vt)
    if row_ptr.size != rows + 1:
        raise ValueError("row_ptr must have rows + 1 entries")
    W, T = C.c_uint32(), C.c_uint32()
    _check(L.hspmm_btcf_sizes_cw(dtype, cw, rows, _p(row_ptr), _p(col_idx), C.byref(W), C.byref(T)))
    W, T = W.value, T.value
    rowOffset = np.zeros(W + 1, np.uint32)
    tcA2B = np.empty(T * cw, np.uint32)
    data = np.empty(T * ROW_WINDOW * cw, vt)
    rowIdx = np.empty(W, np.uint32)
    _check(L.hspmm_btcf_fill_cw(dtype, cw, rows, _p(row_ptr), _p(col_idx), _p(values), int(transpose),
                                _p(rowOffset), _p(tcA2B), _p(data), _p(rowIdx)))
    return dict(rows=rows, cols=cols, nnzs=int(col_idx.size), dtype=dtype, cw=cw, transposed=bool(transpose),
                total_row_windows=(rows + ROW_WINDOW - 1) // ROW_WINDOW, eff_row_windows=W,
                total_tiles=T, rowOffset=rowOffset, tcA2B=tcA2B, data=data, rowIdx=rowIdx)



def btcf_relayout(btcf):
    """Tiles in the layout of one of the reference's build switches (btcf["cw"] = 4 for fp32 storage:
    -DMMA_M16N8K4, src/common.h:28-35; btcf["transposed"]: -DSPARSE_A_TRANSPOSE,
    src/utils/convert.h:207-209) as default tiles; host only."""
    L = load_library()
    dtype = int(btcf["dtype"])
    vt = _val_dtype(dtype)
    cw_default = 8 if dtype == TF32 else 16
    W = int(btcf["eff_row_windows"])
    ro = np.ascontiguousarray(btcf["rowOffset"], np.uint32)
    a2b = np.ascontiguousarray(btcf["tcA2B"], np.uint32)
    data = np.ascontiguousarray(btcf["data"], vt)
    cw = int(btcf.get("cw", cw_default))
    if a2b.size != int(btcf["total_tiles"]) * cw or data.size != a2b.size * ROW_WINDOW or ro.size != W + 1:
        raise ValueError("array sizes do not match eff_row_windows / total_tiles / cw")
    T = C.c_uint32()
    _check(L.hspmm_btcf_relayout_sizes(dtype, cw, W, _p(ro), _p(a2b), C.byref(T)))
    T = T.value
    n_ro = np.empty(W + 1, np.uint32)
    n_a2b = np.empty(T * cw_default, np.uint32)
    n_data = np.empty(T * ROW_WINDOW * cw_default, vt)
    _check(L.hspmm_btcf_relayout_fill(dtype, cw, int(bool(btcf.get("transposed"))), W, _p(ro), _p(a2b), _p(data),
                                      _p(n_ro), _p(n_a2b), _p(n_data)))
    out = dict(btcf)
    out.update(cw=cw_default, transposed=False, total_tiles=T, rowOffset=n_ro, tcA2B=n_a2b, data=n_data)
    return out


BITS_PER_TILE = 0       # HSPMM_BITS_PER_TILE: every tile owns its bitmap words
BITS_AS_REFERENCE = 1   # HSPMM_BITS_AS_REFERENCE: word index as written in src/utils/convert.h:96-101


def csr_to_bitmap(rows, cols, row_ptr, col_idx, values, dtype, transpose=False, bit_layout=BITS_PER_TILE):
    """CSR2BTCF of the reference (src/utils/convert.h:22): returns the BTCF_MTX
    fields (src/utils/class.h:55-67) as a dict of numpy arrays."""
    L = load_library()
    vt = _val_dtype(dtype)
    cw = 8 if dtype == TF32 else 16
    words = 1 if dtype == TF32 else 2
    row_ptr = np.ascontiguousarray(row_ptr, np.uint32)
    col_idx = np.ascontiguousarray(col_idx, np.uint32)
    values = np.ascontiguousarray(values, vt)
    if row_ptr.size != rows + 1:
        raise ValueError("row_ptr must have rows + 1 entries")
    W, T, S = C.c_uint32(), C.c_uint32(), C.c_uint32()
    _check(L.hspmm_bitmap_sizes(dtype, rows, _p(row_ptr), _p(col_idx), C.byref(W), C.byref(T), C.byref(S)))
    W, T, S = W.value, T.value, S.value
    rowOffset = np.zeros(W + 1, np.uint32)
    nnzOffset = np.zeros(T + 1, np.uint32)
    tcA2B = np.empty(T * cw, np.uint32)
    tcBit = np.empty(T * words, np.uint64)
    data = np.empty(S, vt)
    rowIdx = np.empty(W, np.uint32)
    _check(L.hspmm_bitmap_fill(dtype, rows, _p(row_ptr), _p(col_idx), _p(values), int(transpose), int(bit_layout),
                               rowOffset.ctypes.data_as(C.c_void_p), nnzOffset.ctypes.data_as(C.c_void_p),
                               _p(tcA2B), _p(tcBit), _p(data), _p(rowIdx)))
    return dict(rows=rows, cols=cols, nnzs=int(col_idx.size), dtype=dtype, cw=cw,
                total_row_windows=(rows + ROW_WINDOW - 1) // ROW_WINDOW, eff_row_windows=W,
                total_tiles=T, rowOffset=rowOffset, nnzOffset=nnzOffset, tcA2B=tcA2B, tcBit=tcBit,
                data=data, rowIdx=rowIdx)


def bitmap_expand(bitmap):
    """Bitmap tiles -> the dense tiles of the uncompressed format (a BTCF_MTX_NO_BITMAP dict)."""
    L = load_library()
    dtype = bitmap["dtype"]
    vt = _val_dtype(dtype)
    cw = 8 if dtype == TF32 else 16
    T = int(bitmap["total_tiles"])
    nnzOffset = np.ascontiguousarray(bitmap["nnzOffset"], np.uint32)
    tcBit = np.ascontiguousarray(bitmap["tcBit"], np.uint64)
    packed = np.ascontiguousarray(bitmap["data"], vt)
    dense = np.empty(T * ROW_WINDOW * cw, vt)
    _check(L.hspmm_bitmap_expand(dtype, T, _p(nnzOffset), _p(tcBit), _p(packed), _p(dense)))
    out = {k: bitmap[k] for k in ("rows", "cols", "nnzs", "dtype", "total_row_windows", "eff_row_windows",
                                  "total_tiles", "rowOffset", "tcA2B", "rowIdx")}
    out["cw"] = cw
    out["data"] = dense
    return out


def bitmap_to_grouped(bitmap, min_len=32):
    """BTCF2GBTCF of the reference (src/utils/convert.h:232): returns the GBTCF_MTX
    fields (src/utils/class.h:93-108); the tile arrays are shared with `bitmap`."""
    L = load_library()
    rowOffset = np.ascontiguousarray(bitmap["rowOffset"], np.uint32)
    rowIdx = np.ascontiguousarray(bitmap["rowIdx"], np.uint32)
    W = int(bitmap["eff_row_windows"])
    tgl, n = C.c_uint32(), C.c_uint32()
    _check(L.hspmm_group_sizes(W, _p(rowOffset), min_len, C.byref(tgl), C.byref(n)))
    n = n.value
    groupOffset = np.zeros(n + 1, np.uint32)
    groupRowIdx = np.zeros(n, np.uint32)
    atomic = np.zeros(n, np.uint8)
    _check(L.hspmm_group_fill(W, _p(rowOffset), _p(rowIdx), tgl.value,
                              groupOffset.ctypes.data_as(C.c_void_p), _p(groupRowIdx), _p(atomic)))
    out = {k: bitmap[k] for k in ("rows", "cols", "nnzs", "dtype", "cw", "nnzOffset", "tcA2B", "tcBit", "data")}
    # the reference sets both window counts to groupOffset.size() (convert.h:267-268)
    out.update(total_groups=n, tgl=tgl.value, groupOffset=groupOffset, rowIdx=groupRowIdx, atomic=atomic,
               total_row_windows=n + 1, eff_row_windows=n + 1)
    return out


def partition_preview_aligned(rowOffset, group):
    """The partition for plans whose units are all long: every window cut into `group` ranges that
    one workgroup walks (host only).  Ranges have six words; the sixth is 2."""
    L = load_library()
    rowOffset = np.ascontiguousarray(rowOffset, np.uint32)
    W = rowOffset.size - 1
    n = C.c_uint32()
    _check(L.hspmm_partition_preview_aligned(W, _p(rowOffset), group, None, 0, C.byref(n)))
    ranges = np.zeros((n.value, 6), np.uint32)
    _check(L.hspmm_partition_preview_aligned(W, _p(rowOffset), group, _p(ranges), n.value, None))
    return ranges


def partition_preview(rowOffset, target_ranges, group=1, group_offset=None):
    """The work partition hspmm_create would build (host only).  group > 1: the partition
    for workgroups whose waves add the partial sums of one window among themselves
    (ranges then have a sixth word, "combine").  group_offset: the ends of the caller's groups
    (GBTCF_MTX.groupOffset); windows are then cut only there (set_group_cuts(1))."""
    L = load_library()
    rowOffset = np.ascontiguousarray(rowOffset, np.uint32)
    W = rowOffset.size - 1
    n, ns, nslots = C.c_uint32(), C.c_uint32(), C.c_uint32()
    if group_offset is not None:
        go = np.ascontiguousarray(group_offset, np.uint32)
        _check(L.hspmm_partition_preview_group_cuts(W, _p(rowOffset), target_ranges, go.size - 1, _p(go), None, 0,
                                                    C.byref(n), C.byref(ns), C.byref(nslots)))
        ranges = np.zeros((n.value, 5), np.uint32)
        _check(L.hspmm_partition_preview_group_cuts(W, _p(rowOffset), target_ranges, go.size - 1, _p(go), _p(ranges),
                                                    n.value, None, None, None))
    elif group == 1:
        _check(L.hspmm_partition_preview(W, _p(rowOffset), target_ranges, None, 0, C.byref(n), C.byref(ns),
                                         C.byref(nslots)))
        ranges = np.zeros((n.value, 5), np.uint32)
        _check(L.hspmm_partition_preview(W, _p(rowOffset), target_ranges, _p(ranges), n.value, None, None, None))
    else:
        _check(L.hspmm_partition_preview_grouped(W, _p(rowOffset), target_ranges, group, None, 0, C.byref(n),
                                                 C.byref(ns), C.byref(nslots)))
        ranges = np.zeros((n.value, 6), np.uint32)
        _check(L.hspmm_partition_preview_grouped(W, _p(rowOffset), target_ranges, group, _p(ranges), n.value, None,
                                                 None, None))
    return dict(ranges=ranges, n_split_windows=ns.value, n_partial_slots=nslots.value)


def panel_units_preview(btcf, max_windows=4):
    """How the LDS-staging kernels built on the 16-bit MFMA group adjacent windows into units
    (host only): dict with group_first, group_count and the rewritten matrix (rowOffset, tcA2B,
    data, total_tiles) whose windows carry their group's union of column lists."""
    L = load_library()
    dtype = btcf["dtype"]
    vt = _val_dtype(dtype)
    cw = 8 if dtype == TF32 else 16
    ro = np.ascontiguousarray(btcf["rowOffset"], np.uint32)
    a2b = np.ascontiguousarray(btcf["tcA2B"], np.uint32)
    data = np.ascontiguousarray(btcf["data"], vt)
    ri = np.ascontiguousarray(btcf["rowIdx"], np.uint32)
    W, T = int(btcf["eff_row_windows"]), int(btcf["total_tiles"])
    ng, nt = C.c_uint32(), C.c_uint32()
    first = np.zeros(max(W, 1), np.uint32)
    count = np.zeros(max(W, 1), np.uint32)
    new_ro = np.zeros(W + 1, np.uint32)
    args = (dtype, int(btcf["rows"]), int(btcf["cols"]), W, T, _p(ro), _p(a2b), _p(data), _p(ri), max_windows)
    _check(L.hspmm_panel_units_preview(*args, C.byref(ng), _p(first), _p(count), _p(new_ro), C.byref(nt), 0, None, None))
    new_a2b = np.zeros(nt.value * cw, np.uint32)
    new_data = np.zeros(nt.value * 8 * cw, vt)
    _check(L.hspmm_panel_units_preview(*args, None, None, None, None, None, nt.value, _p(new_a2b), _p(new_data)))
    return dict(group_first=first[:ng.value].copy(), group_count=count[:ng.value].copy(), rowOffset=new_ro,
                tcA2B=new_a2b, data=new_data, total_tiles=nt.value)


class Plan:
    """Device-resident A plus its work partition (hspmm_create / hspmm_destroy)."""

    def __init__(self, btcf):
        """btcf: a dict as returned by csr_to_btcf (uncompressed tiles), csr_to_bitmap
        (it has "tcBit") or bitmap_to_grouped (it has "groupOffset")."""
        L = load_library()
        self._h = C.c_void_p()
        self.dtype = btcf["dtype"]
        self.rows, self.cols = int(btcf["rows"]), int(btcf["cols"])
        vt = _val_dtype(self.dtype)
        a2b = np.ascontiguousarray(btcf["tcA2B"], np.uint32)
        data = np.ascontiguousarray(btcf["data"], vt)
        ri = np.ascontiguousarray(btcf["rowIdx"], np.uint32)
        if "groupOffset" in btcf:
            go = np.ascontiguousarray(btcf["groupOffset"], np.uint32)
            no = np.ascontiguousarray(btcf["nnzOffset"], np.uint32)
            bits = np.ascontiguousarray(btcf["tcBit"], np.uint64)
            at = np.ascontiguousarray(btcf["atomic"], np.uint8)
            _check(L.hspmm_create_grouped(C.byref(self._h), self.dtype, self.rows, self.cols,
                                          int(btcf["total_groups"]), go.ctypes.data_as(C.c_void_p), _p(no), _p(a2b),
                                          _p(bits), _p(data), _p(ri), _p(at)))
            return
        ro = np.ascontiguousarray(btcf["rowOffset"], np.uint32)
        if "tcBit" in btcf:
            no = np.ascontiguousarray(btcf["nnzOffset"], np.uint32)
            bits = np.ascontiguousarray(btcf["tcBit"], np.uint64)
            _check(L.hspmm_create_bitmap(C.byref(self._h), self.dtype, self.rows, self.cols,
                                         int(btcf["eff_row_windows"]), int(btcf["total_tiles"]),
                                         _p(ro), _p(no), _p(a2b), _p(bits), _p(data), _p(ri)))
            return
        cw_default = 8 if self.dtype == TF32 else 16
        if btcf.get("transposed") or int(btcf.get("cw", cw_default)) != cw_default:
            # tiles in the order of -DSPARSE_A_TRANSPOSE and / or the 8 x 4 tiles of -DMMA_M16N8K4
            _check(L.hspmm_create_layout(C.byref(self._h), self.dtype, int(btcf.get("cw", 0)),
                                         int(bool(btcf.get("transposed"))), self.rows, self.cols,
                                         int(btcf["eff_row_windows"]), int(btcf["total_tiles"]),
                                         _p(ro), _p(a2b), _p(data), _p(ri)))
            return
        _check(L.hspmm_create(C.byref(self._h), self.dtype, self.rows, self.cols,
                              int(btcf["eff_row_windows"]), int(btcf["total_tiles"]),
                              _p(ro), _p(a2b), _p(data), _p(ri)))

    def run(self, dB_ptr, dC_ptr, N, stream=0):
        """dB_ptr / dC_ptr: integer device addresses (e.g. torch tensor .data_ptr())."""
        _check(load_library().hspmm_run(self._h, C.c_void_p(dB_ptr), C.c_void_p(dC_ptr), N, C.c_void_p(stream)))

    def run_static(self, dB_ptr, dC_ptr, N, stream=0):
        """hspmm_run_static: the same launch with its partial sums in the library's fixed device array
        (no allocation; the partition for N must exist: prepare(N) or one run with N first)."""
        _check(load_library().hspmm_run_static(self._h, C.c_void_p(dB_ptr), C.c_void_p(dC_ptr), N,
                                               C.c_void_p(stream)))

    def prepare(self, N):
        """hspmm_prepare: builds what the first run with feature dimension N would build; launches nothing."""
        _check(load_library().hspmm_prepare(self._h, N))

    def bench(self, dB_ptr, dC_ptr, N, warmup=3, runs=5, stream=0):
        """Total milliseconds of `runs` launches (WARMUP_RUNS / RUNS, src/common.h:48-49)."""
        ms = C.c_float()
        _check(load_library().hspmm_bench(self._h, C.c_void_p(dB_ptr), C.c_void_p(dC_ptr), N, warmup, runs,
                                          C.c_void_p(stream), C.byref(ms)))
        return ms.value

    def profile(self, dB_ptr, dC_ptr, N, runs=5, stream=0):
        """(main kernel ms, partial-sum kernel ms), totals over `runs` launches."""
        a, b = C.c_float(), C.c_float()
        _check(load_library().hspmm_profile(self._h, C.c_void_p(dB_ptr), C.c_void_p(dC_ptr), N, runs,
                                            C.c_void_p(stream), C.byref(a), C.byref(b)))
        return a.value, b.value

    def measure_gather(self, dB_ptr, N, runs=5, stream=0):
        """(ms per run, bytes loaded per run) of the plan's row gathers alone (measurement only)."""
        ms, nbytes = C.c_float(), C.c_uint64()
        _check(load_library().hspmm_measure_gather(self._h, C.c_void_p(dB_ptr), N, runs, C.c_void_p(stream),
                                                   C.byref(ms), C.byref(nbytes)))
        return ms.value, nbytes.value

    def partition_as_groups(self):
        """hspmm_partition_as_groups: the plan's balanced partition as the group arrays of a GBTCF_MTX
        (groupOffset, rowIdx per group, atomic) over the tile arrays the plan was made from."""
        L = load_library()
        n = C.c_uint32()
        _check(L.hspmm_partition_as_groups(self._h, 0, C.byref(n), None, None, None))
        n = n.value
        groupOffset = np.zeros(n + 1, np.uint32)
        rowIdx = np.zeros(n, np.uint32)
        atomic = np.zeros(n, np.uint8)
        _check(L.hspmm_partition_as_groups(self._h, n, C.byref(C.c_uint32()), _p(groupOffset), _p(rowIdx), _p(atomic)))
        return dict(total_groups=n, groupOffset=groupOffset, rowIdx=rowIdx, atomic=atomic)

    def info(self):
        inf = PlanInfo()
        _check(load_library().hspmm_get_plan_info(self._h, C.byref(inf)))
        return {k: getattr(inf, k) for k, _ in PlanInfo._fields_}

    def partition(self):
        n = self.info()["n_ranges"]
        ranges = np.zeros((n, 5), np.uint32)
        if n:
            _check(load_library().hspmm_get_partition(self._h, _p(ranges), n))
        return ranges

    def close(self):
        if self._h:
            load_library().hspmm_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
