"""The C-ABI library loads without a GPU and exports every symbol that
include/hspmm.h declares; host-only entry points behave (no device calls here)."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hspmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hspmm_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(hs):
    lib = ctypes.CDLL(hs.library_path())
    names = declared_symbols()
    assert len(names) >= 14 and "hspmm_create" in names and "hspmm_run" in names
    for n in names:
        assert hasattr(lib, n), n


def test_nothing_but_the_declared_c_abi_is_exported(hs):
    # the dynamic symbol table of the library, defined symbols only
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", hs.library_path()], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == declared_symbols()


def test_no_torch_types_in_the_header():
    text = open(os.path.join(ROOT, "include", "hspmm.h")).read()
    assert "torch" not in text and "at::" not in text and 'extern "C"' in text


def test_scheduler_knobs_round_trip(hs):
    # Scheduler::configure / getters of the reference (src/scheduler.h:26-41)
    assert hs.get_config() == (0, 0, 0, 0)
    hs.configure(4, 2, 3, 128)
    assert hs.get_config() == (4, 2, 3, 128)
    for bad in ((5, 0, 0, 0), (9, 0, 0, 0), (0, 5, 0, 0), (0, 0, 17, 0), (-1, 0, 0, 0), (0, 0, 0, -3)):
        with pytest.raises(hs.HspmmError):
            hs.configure(*bad)
    assert hs.get_config() == (4, 2, 3, 128)
    hs.configure()
    assert hs.get_config() == (0, 0, 0, 0)
    with pytest.raises(hs.HspmmError):
        hs.set_kernel_mode(9)
    hs.set_kernel_mode(0)


def test_create_rejects_malformed_formats_before_touching_the_device(hs):
    ok = dict(rows=16, cols=40, dtype=0, eff_row_windows=2, total_tiles=2,
              rowOffset=np.array([0, 1, 2], np.uint32), rowIdx=np.array([0, 8], np.uint32),
              tcA2B=np.concatenate([np.arange(16), np.arange(16) + 3]).astype(np.uint32),
              data=np.zeros(2 * 128, np.uint16))
    def broken(**kw):
        d = dict(ok); d.update(kw); return d
    cases = [
        broken(rowOffset=np.array([1, 2, 3], np.uint32)),
        broken(rowOffset=np.array([0, 1, 1], np.uint32)),
        broken(rowOffset=np.array([0, 1, 3], np.uint32)),
        broken(rowIdx=np.array([0, 4], np.uint32)),
        broken(rowIdx=np.array([8, 0], np.uint32)),
        broken(rowIdx=np.array([0, 16], np.uint32)),
        broken(tcA2B=np.concatenate([np.arange(16), np.arange(16) + 30]).astype(np.uint32)),
        broken(tcA2B=np.concatenate([[0xFFFFFFFF], np.arange(31)]).astype(np.uint32)),
        broken(tcA2B=np.concatenate([[0, 0xFFFFFFFF, 5], np.arange(29)]).astype(np.uint32)),
        broken(eff_row_windows=3, rowOffset=np.array([0, 1, 2, 3], np.uint32), rowIdx=np.array([0, 8, 16], np.uint32), total_tiles=3),
    ]
    for c in cases:
        with pytest.raises(hs.HspmmError) as e:
            hs.Plan(c)
        assert e.value.code in (1,), str(e.value)        # HSPMM_ERR_INVALID, raised by host-side validation
    L = hs.load_library()
    h = ctypes.c_void_p()
    assert L.hspmm_create(ctypes.byref(h), 3, 8, 8, 0, 0, None, None, None, None) == 1   # unknown dtype
    assert b"dtype" in L.hspmm_last_error() and not h.value


def test_validation_on_all_cores_names_the_first_bad_tile(hs):
    # 200 000 tiles (the check runs on worker threads from 65 536 tiles per worker on): two bad tiles planted
    W, per = 25000, 8
    T = W * per
    ids = np.tile(np.arange(per * 16, dtype=np.uint32), W)
    ids[150000 * 16 + 3] = 5000                             # column id >= cols
    ids[70000 * 16 + 1] = 0xFFFFFFFF                        # a real id behind padding
    fmt = dict(rows=W * 8, cols=per * 16, dtype=0, eff_row_windows=W, total_tiles=T,
               rowOffset=(np.arange(W + 1) * per).astype(np.uint32), rowIdx=(np.arange(W) * 8).astype(np.uint32),
               tcA2B=ids, data=np.zeros(T * 128, np.uint16))
    with pytest.raises(hs.HspmmError) as e:
        hs.Plan(fmt)
    assert e.value.code == 1 and "tile 70000:" in str(e.value), str(e.value)


def test_bitmap_and_grouped_plans_reject_malformed_arrays_before_touching_the_device(hs):
    from util import random_csr
    rng = np.random.default_rng(21)
    A = random_csr(rng, 64, 900, 0.2, 0, 0.0, heavy_rows=(3,))
    b = hs.csr_to_bitmap(64, 900, A["row_ptr"], A["col_idx"], A["values"], 0)
    g = hs.bitmap_to_grouped(b, min_len=4)
    assert g["atomic"].any() and not g["atomic"].all()

    def broken(src, **kw):
        d = dict(src)
        for k, f in kw.items():
            a = src[k].copy()
            f(a)
            d[k] = a
        return d

    def flip(a): a[5] ^= np.uint64(2)
    def shift(a): a[2] += 1
    def flag_one(a): a[int(np.argmax(g["atomic"] == 0))] = 1
    def flag_zero(a): a[int(np.argmax(g["atomic"] == 1))] = 0
    def stall(a): a[3] = a[2]
    def scatter(a): a[-1] = a[0]
    cases = [broken(b, tcBit=flip), broken(b, nnzOffset=shift), broken(g, tcBit=flip), broken(g, atomic=flag_one),
             broken(g, atomic=flag_zero), broken(g, groupOffset=stall), broken(g, rowIdx=scatter)]
    for c in cases:
        with pytest.raises(hs.HspmmError) as e:
            hs.Plan(c)
        assert e.value.code == 1, str(e.value)           # HSPMM_ERR_INVALID from host-side checks


def test_operator_fails_loudly_without_a_gfx950_device(hs):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    ok = dict(rows=8, cols=16, dtype=0, eff_row_windows=1, total_tiles=1,
              rowOffset=np.array([0, 1], np.uint32), rowIdx=np.array([0], np.uint32),
              tcA2B=np.arange(16).astype(np.uint32), data=np.zeros(128, np.uint16))
    with pytest.raises(hs.HspmmError) as e:
        hs.Plan(ok)
    assert e.value.code == 2                              # HSPMM_ERR_DEVICE: no CPU fallback exists


def test_static_scratch_array_is_a_visible_symbol_of_the_device_code(hs):
    """hspmm_run_static finds its fixed device array with hipGetSymbolAddress, which looks the array up
    by name in the gfx950 code object: the symbol must be there with global binding (a file-scope
    static that the compiler leaves local, e.g. one marked `used`, cannot be found at run time)."""
    import shutil
    import subprocess
    import tempfile
    tools = "/opt/rocm/llvm/bin"
    obj = os.path.join(ROOT, "hopper_spmm_amd", "csrc", "build", "hspmm_run.hip.o")
    if not (os.path.exists(obj) and shutil.which(os.path.join(tools, "clang-offload-bundler"))):
        pytest.skip("needs the object file of the last build and the ROCm llvm tools")
    with tempfile.TemporaryDirectory() as d:
        fat, dev = os.path.join(d, "fatbin"), os.path.join(d, "dev.o")
        subprocess.check_call([os.path.join(tools, "llvm-objcopy"), "--dump-section", ".hip_fatbin=" + fat, obj])
        subprocess.check_call([os.path.join(tools, "clang-offload-bundler"), "--unbundle", "--type=o", "--input=" + fat,
                               "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", "--output=" + dev])
        table = subprocess.check_output([os.path.join(tools, "llvm-readelf"), "-s", dev], text=True)
    rows = [l.split() for l in table.splitlines() if "hspmm_static_scratch" in l]
    assert rows, "the static scratch array is not in the device code object"
    assert all(r[4] == "GLOBAL" and int(r[2]) == 32 << 20 for r in rows), rows
