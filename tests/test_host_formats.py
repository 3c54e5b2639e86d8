"""The product's host format functions (hspmm_mtx_load, hspmm_btcf_sizes/fill in
libhspmm.so) against the pinned oracle and the golden vectors (hand-checkable definition cases of the reference converters).
Bit-exact: this is integer / byte work."""
import json
import os

import numpy as np
import pytest

from util import random_csr

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DT = {0: "fp16", 1: "tf32", 2: "bf16"}


def _same_btcf(a, b):
    for k in ("eff_row_windows", "total_tiles", "total_row_windows"):
        assert a[k] == b[k], k
    for k in ("rowOffset", "tcA2B", "rowIdx"):
        assert np.array_equal(a[k], b[k]), k
    assert a["data"].tobytes() == b["data"].tobytes()


def test_golden_vectors_through_the_library(hs):
    with open(os.path.join(GOLD, "expected.json")) as f:
        G = json.load(f)
    for name in ("tiny", "gap"):
        g = G[name]
        dt = 0 if g["dtype"] == "fp16" else 1
        m = hs.mtx_load(os.path.join(GOLD, g["file"]), dt)
        assert (m["rows"], m["cols"], m["nnzs"]) == (g["rows"], g["cols"], g["nnzs"])
        b = hs.csr_to_btcf(m["rows"], m["cols"], m["row_ptr"], m["col_idx"], m["values"], dt)
        assert b["total_row_windows"] == g["total_row_windows"]
        assert b["eff_row_windows"] == g["eff_row_windows"] and b["total_tiles"] == g["total_tiles"]
        assert b["data"].size == g["data_size"]
        assert b["rowOffset"].tolist() == g["rowOffset"]
        assert b["rowIdx"].tolist() == g["rowIdx"]
        assert b["tcA2B"].tolist() == g["tcA2B"]
        if "tile_nonzeros" in g:
            want = np.zeros((g["total_tiles"], 8, b["cw"]), np.float32)
            for t, r, k, v in g["tile_nonzeros"]:
                want[t, r, k] = v
            assert np.array_equal(b["data"].view(np.float16).astype(np.float32).reshape(want.shape), want)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_loader_equals_oracle(hs, oracle, tmp_path, dtype):
    rng = np.random.default_rng(100 + dtype)
    for case in range(6):
        rows, cols = int(rng.integers(1, 200)), int(rng.integers(1, 200))
        nnz = int(rng.integers(0, min(rows * cols, 3000) + 1))
        flat = rng.choice(rows * cols, size=nnz, replace=False)
        r, c = flat // cols, flat % cols
        v = rng.normal(size=nnz) * 10.0 ** rng.integers(-9, 6, nnz)
        p = tmp_path / ("m%d.mtx" % case)
        with open(p, "w") as f:
            f.write("%%MatrixMarket matrix coordinate real general\n%comment line\n%\n")
            f.write("%d %d %d\n" % (rows, cols, nnz))
            for i in range(nnz):
                if case == 1 and i % 17 == 3:
                    f.write("this line is skipped\n")
                sep = "\t" if case == 2 else " "
                f.write("%d%s%d%s%.9g\n" % (r[i] + 1, sep, c[i] + 1, sep, v[i]))
        a = hs.mtx_load(str(p), dtype)
        o = oracle.mtx_read(str(p), DT[dtype])
        assert (a["rows"], a["cols"], a["nnzs"]) == (o["rows"], o["cols"], o["nnzs"])
        assert np.array_equal(a["row_ptr"], o["row_ptr"])
        assert np.array_equal(a["col_idx"], o["col_idx"])
        assert a["values"].tobytes() == o["values"].tobytes()


def test_loader_special_values_and_short_files(hs, oracle, tmp_path):
    p = tmp_path / "s.mtx"
    p.write_text("%%MatrixMarket\n4 4 9\n1 1 65520\n1 2 1e-8\n2 2 -6.1e-5\n2 3 5.96e-8\n"
                 "3 1 inf\n3 3 0x1.8p1\n4 4 2.98e-8\n4 1 1e39\n")
    for dt in (0, 1):
        a = hs.mtx_load(str(p), dt)
        o = oracle.mtx_read(str(p), DT[dt])
        assert a["nnzs"] == o["nnzs"] == 8 and o["declared_nnz"] == 9        # load.h:234-238
        assert np.array_equal(a["row_ptr"], o["row_ptr"]) and np.array_equal(a["col_idx"], o["col_idx"])
        assert a["values"].tobytes() == o["values"].tobytes()


def test_loader_number_forms_equal_the_c_library(hs, oracle, tmp_path):
    """The loader's own number parsing against sscanf (the oracle reads with it):
    digit counts on both sides of what fits a double exactly, exponents on both sides
    of 10^22, ties between two floats, subnormal and overflowing values, signs,
    hexadecimal, inf and nan, indices with signs and beyond 32 bits."""
    rng = np.random.default_rng(77)
    vals = ["0", "-0", "+0.0", ".5", "5.", "-.25e1", "+1.5E+3", "1e", "1e+", "2.5e-3x", "inf", "-inf", "nan", "INFINITY",
            "0x1p3", "0x1.8p-2", "1e-42", "1e-46", "3.4028235e38", "3.4028236e38", "1e40", "-1e40",
            "16777217", "16777217.0000000001", "9007199254740993", "0.1", "123456789012345678901234567890",
            "0.000000000000000000000000000001", "1e22", "1e23", "8.5e-23", "1.17549435e-38", "1.17549421e-38"]
    for _ in range(3000):
        nd = int(rng.integers(1, 26))
        digits = "".join(rng.choice(list("0123456789"), nd))
        point = int(rng.integers(0, nd + 1))
        txt = digits[:point] + "." + digits[point:] if rng.random() < 0.7 else digits
        if rng.random() < 0.6:
            txt += "e%d" % int(rng.integers(-45, 40))
        vals.append(("-" if rng.random() < 0.3 else "") + txt)
    # exact ties: the midpoint of two neighbouring floats, written out in full
    f = np.abs(rng.normal(size=400).astype(np.float32)) * np.float32(10.0) ** rng.integers(-8, 9, 400).astype(np.float32)
    mid = (f.astype(np.float64) + np.nextafter(f, np.float32(np.inf)).astype(np.float64)) / 2
    from decimal import Decimal
    for m in mid:
        d = Decimal(float(m))
        vals += [format(d, "f"), format(d + d * Decimal(10) ** -25, "f"), format(d - d * Decimal(10) ** -25, "f")]
    rows = len(vals)
    p = tmp_path / "forms.mtx"
    with open(p, "w") as fh:
        fh.write("%d %d %d\n" % (rows, 7, rows + 6))
        for i, v in enumerate(vals):
            fh.write("%d %d %s\n" % (i + 1, 1 + i % 7, v))
        fh.write("+3 +2 1.5\n1 -4294967294 2.5\n4294967297 4294967298 3.5\n")   # signs and wrap-around: (3,2) (1,2) (1,2)
        fh.write("2 x 1\n2 3\n 5\t6\t7.5 trailing words\n")
    for dt in (1, 0):
        a = hs.mtx_load(str(p), dt)
        o = oracle.mtx_read(str(p), DT[dt])
        assert a["nnzs"] == o["nnzs"] and a["nnzs"] >= rows
        assert np.array_equal(a["row_ptr"], o["row_ptr"]) and np.array_equal(a["col_idx"], o["col_idx"])
        assert a["values"].tobytes() == o["values"].tobytes()


def test_loader_blocks_of_a_large_file_equal_the_oracle(hs, oracle, tmp_path):
    # several megabytes, so that the data lines are parsed in more than one block; a few
    # over-long lines (cut into 1023-character pieces like fgets does) and blank lines
    rng = np.random.default_rng(78)
    rows, cols, nnz = 3000, 2500, 400000
    flat = rng.choice(rows * cols, size=nnz, replace=False)
    v = rng.normal(size=nnz)
    p = tmp_path / "big.mtx"
    with open(p, "w") as fh:
        fh.write("%%MatrixMarket matrix coordinate real general\n%d %d %d\n" % (rows, cols, nnz))
        for i in range(nnz):
            if i % 50021 == 7:
                fh.write(" " * 2500 + "\n")
            if i % 70001 == 11:
                fh.write("\n")
            fh.write("%d %d %.8g\n" % (flat[i] // cols + 1, flat[i] % cols + 1, v[i]))
    assert os.path.getsize(p) > 6 << 20
    a = hs.mtx_load(str(p), 0)
    o = oracle.mtx_read(str(p), "fp16")
    assert a["nnzs"] == o["nnzs"] == nnz
    assert np.array_equal(a["row_ptr"], o["row_ptr"]) and np.array_equal(a["col_idx"], o["col_idx"])
    assert a["values"].tobytes() == o["values"].tobytes()


def test_loader_errors(hs, tmp_path):
    with pytest.raises(hs.HspmmError) as e:
        hs.mtx_load(str(tmp_path / "nope.mtx"), 0)
    assert e.value.code == 4 and "cannot open" in str(e.value)               # load.h:176-180
    bad = tmp_path / "bad.mtx"
    bad.write_text("%%MatrixMarket\n% only comments\n")
    with pytest.raises(hs.HspmmError) as e:
        hs.mtx_load(str(bad), 0)
    assert e.value.code == 4                                                 # load.h:190-194
    oob = tmp_path / "oob.mtx"
    oob.write_text("2 2 1\n3 1 1.0\n")
    with pytest.raises(hs.HspmmError):
        hs.mtx_load(str(oob), 1)
    with pytest.raises(hs.HspmmError):
        hs.mtx_load(str(oob), 7)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_converter_equals_oracle(hs, oracle, dtype):
    rng = np.random.default_rng(200 + dtype)
    shapes = [(1, 1, 1.0, 0.0), (8, 16, 0.5, 0.0), (9, 17, 0.5, 0.0), (27, 12, 0.1, 0.7), (64, 500, 0.05, 0.3),
              (203, 77, 0.3, 0.1), (1000, 1000, 0.004, 0.5), (16, 4000, 0.6, 0.0)]
    for rows, cols, dens, erp in shapes:
        A = random_csr(rng, rows, cols, dens, dtype, erp)
        for tr in (False, True):
            a = hs.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype, transpose=tr)
            o = oracle.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], DT[dtype], transpose=tr)
            _same_btcf(a, o)


def test_converter_writes_the_8_by_4_tiles_of_the_m16n8k4_build(hs, oracle):
    """CSR2BTCFNOBITMAP with COL_WINDOW 4 (the reference's -DMMA_M16N8K4 build of the tf32 variant,
    src/common.h:28-35), row by row and column by column: the library's converter against the oracle's,
    bit for bit; the width is refused for the 16-bit types."""
    rng = np.random.default_rng(270)
    shapes = [(1, 1, 1.0, 0.0), (8, 4, 1.0, 0.0), (9, 5, 0.5, 0.0), (27, 12, 0.1, 0.7), (64, 500, 0.05, 0.3),
              (203, 77, 0.3, 0.1), (1000, 1000, 0.004, 0.5), (16, 4000, 0.6, 0.0)]
    for rows, cols, dens, erp in shapes:
        A = random_csr(rng, rows, cols, dens, 1, erp)
        for tr in (False, True):
            a = hs.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], 1, transpose=tr, cw=4)
            o = oracle.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], "tf32", transpose=tr, cw=4)
            assert a["cw"] == 4 and a["tcA2B"].size == 4 * a["total_tiles"] and a["data"].size == 32 * a["total_tiles"]
            _same_btcf(a, o)
    A = random_csr(rng, 16, 40, 0.3, 0)
    with pytest.raises(hs.HspmmError):
        hs.csr_to_btcf(16, 40, A["row_ptr"], A["col_idx"], A["values"], 0, cw=4)
    with pytest.raises(hs.HspmmError):
        hs.csr_to_btcf(16, 40, A["row_ptr"], A["col_idx"], A["values"].astype(np.float32), 1, cw=16)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_relayout_of_the_build_switch_formats_gives_the_default_tiles(hs, oracle, dtype):
    """Tiles written with -DSPARSE_A_TRANSPOSE (convert.h:207-209) and, for fp32 storage, the
    8 x 4 tiles of -DMMA_M16N8K4 (common.h:28-35), both from the oracle's converter, re-laid
    out by the library: exactly the arrays the oracle's converter writes without the switches
    (every window's sorted columns, cut into tiles of the default width)."""
    rng = np.random.default_rng(260 + dtype)
    shapes = [(1, 1, 1.0, 0.0), (8, 16, 0.5, 0.0), (9, 17, 0.5, 0.0), (27, 12, 0.1, 0.7), (64, 500, 0.05, 0.3),
              (203, 77, 0.3, 0.1), (1000, 1000, 0.004, 0.5), (16, 4000, 0.6, 0.0)]
    for rows, cols, dens, erp in shapes:
        A = random_csr(rng, rows, cols, dens, dtype, erp)
        csr = (rows, cols, A["row_ptr"], A["col_idx"], A["values"], DT[dtype])
        want = oracle.csr_to_btcf(*csr)
        for cw in ((None, 4) if dtype == 1 else (None,)):
            for tr in (False, True):
                src = dict(oracle.csr_to_btcf(*csr, transpose=tr, cw=cw))
                if cw == 4:
                    assert src["tcA2B"].size == 4 * src["total_tiles"]
                src.update(dtype=dtype, transposed=tr)
                _same_btcf(hs.btcf_relayout(src), want)
    # padding columns between real ones (not what the converter writes, but a valid tile list) are dropped,
    # a window of padding only is refused, and so is a width the element type does not have
    src = dict(rows=8, cols=40, dtype=1, cw=4, transposed=True, eff_row_windows=1, total_tiles=3,
               rowOffset=np.array([0, 3], np.uint32), rowIdx=np.array([0], np.uint32),
               tcA2B=np.array([7, hs.IDX_MAX, 9, hs.IDX_MAX] + [hs.IDX_MAX] * 4 + [30, 31, 32, 33], np.uint32),
               data=np.arange(96, dtype=np.float32))
    out = hs.btcf_relayout(src)
    assert out["total_tiles"] == 1 and out["tcA2B"].tolist() == [7, 9, 30, 31, 32, 33, hs.IDX_MAX, hs.IDX_MAX]
    tile = out["data"].reshape(8, 8)
    for k, (t, kk) in enumerate([(0, 0), (0, 2), (2, 0), (2, 1), (2, 2), (2, 3)]):
        assert tile[:, k].tolist() == [32 * t + 8 * kk + r for r in range(8)]
    assert not tile[:, 6:].any()
    src["tcA2B"][:] = hs.IDX_MAX
    with pytest.raises(hs.HspmmError):
        hs.btcf_relayout(src)
    with pytest.raises(hs.HspmmError):
        hs.btcf_relayout(dict(src, dtype=0, data=np.zeros(96, np.uint16)))


def test_converter_large_multithreaded_equals_oracle(hs, oracle):
    # big enough that the library's window loop runs on several threads
    from hopper_spmm_amd import generators as G
    A = G.rmat(15, 16, seed=9)
    a = hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], 0)
    o = oracle.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], "fp16")
    _same_btcf(a, o)
    A = G.pruned_weight(1376, 512, 0.1, seed=4)
    a = hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], 1)
    o = oracle.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], "tf32")
    _same_btcf(a, o)


def test_converter_empty_and_duplicates(hs, oracle):
    # no stored entry at all: zero effective windows
    rp = np.zeros(21, np.uint32)
    b = hs.csr_to_btcf(20, 5, rp, np.zeros(0, np.uint32), np.zeros(0, np.uint16), 0)
    assert b["eff_row_windows"] == 0 and b["total_tiles"] == 0 and b["rowOffset"].tolist() == [0]
    # zero rows
    b = hs.csr_to_btcf(0, 5, np.zeros(1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32), 1)
    assert b["eff_row_windows"] == 0 and b["total_row_windows"] == 0
    # duplicate position: the later stored entry stays (convert.h:215)
    rp = np.array([0, 3], np.uint32)
    ci = np.array([4, 4, 9], np.uint32)
    vv = np.array([1.0, 2.0, 3.0], np.float32)
    a = hs.csr_to_btcf(1, 10, rp, ci, vv, 1)
    o = oracle.csr_to_btcf(1, 10, rp, ci, vv, "tf32")
    _same_btcf(a, o)
    assert a["data"][0] == 2.0
    # an explicit zero still claims a tile column
    a = hs.csr_to_btcf(1, 10, np.array([0, 2], np.uint32), np.array([1, 7], np.uint32), np.array([0.0, 5.0], np.float32), 1)
    assert a["tcA2B"].tolist()[:2] == [1, 7]


# ------------------------------------------------------------------ bitmap tiles and groups
@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_bitmap_converter_equals_oracle(hs, oracle, dtype):
    rng = np.random.default_rng(400 + dtype)
    shapes = [(1, 1, 1.0, 0.0), (8, 16, 0.5, 0.0), (9, 17, 0.5, 0.0), (27, 12, 0.1, 0.7), (64, 500, 0.05, 0.3),
              (203, 77, 0.3, 0.1), (1000, 1000, 0.004, 0.5), (16, 4000, 0.6, 0.0)]
    for rows, cols, dens, erp in shapes:
        A = random_csr(rng, rows, cols, dens, dtype, erp)
        for tr in (False, True):
            for layout in (hs.BITS_PER_TILE, hs.BITS_AS_REFERENCE):
                a = hs.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype, tr, layout)
                o = oracle.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], DT[dtype], tr,
                                         layout == hs.BITS_AS_REFERENCE)
                for k in ("rowOffset", "nnzOffset", "tcA2B", "tcBit", "rowIdx"):
                    assert np.array_equal(a[k], o[k]), k
                assert a["data"].tobytes() == o["data"].tobytes()
                assert (a["eff_row_windows"], a["total_tiles"]) == (o["eff_row_windows"], o["total_tiles"])
            # expansion gives back the uncompressed converter's tiles, in both tile orders
            e = hs.bitmap_expand(hs.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype, tr))
            d = hs.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype, transpose=tr)
            _same_btcf(e, d)


def test_bitmap_golden_vector_through_the_library(hs):
    import json
    with open(os.path.join(GOLD, "expected.json")) as f:
        g = json.load(f)["tiny"]
    A = hs.mtx_load(os.path.join(GOLD, "tiny.mtx"), 0)
    b = hs.csr_to_bitmap(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], 0,
                         bit_layout=hs.BITS_AS_REFERENCE)
    assert b["nnzOffset"].tolist() == g["bitmap"]["nnzOffset"]
    assert b["data"].view(np.float16).astype(np.float32).tolist() == g["bitmap"]["data"]
    assert [int(x) for x in b["tcBit"]] == [int(x, 16) for x in g["bitmap"]["tcBit_as_reference"]]


def test_bitmap_large_multithreaded_equals_oracle(hs, oracle):
    from hopper_spmm_amd import generators as G
    A = G.rmat(15, 16, seed=9)
    a = hs.csr_to_bitmap(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], 0)
    o = oracle.csr_to_bitmap(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], "fp16")
    for k in ("rowOffset", "nnzOffset", "tcA2B", "tcBit", "rowIdx"):
        assert np.array_equal(a[k], o[k]), k
    assert a["data"].tobytes() == o["data"].tobytes()
    _same_btcf(hs.bitmap_expand(a), hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], 0))


def test_bitmap_expand_rejects_inconsistent_tiles(hs):
    rng = np.random.default_rng(3)
    A = random_csr(rng, 40, 60, 0.2, 0)
    b = hs.csr_to_bitmap(40, 60, A["row_ptr"], A["col_idx"], A["values"], 0)
    bad = dict(b)
    bad["tcBit"] = b["tcBit"].copy()
    bad["tcBit"][3] ^= np.uint64(1) << np.uint64(63)             # one bit more or less than nnzOffset says
    with pytest.raises(hs.HspmmError) as e:
        hs.bitmap_expand(bad)
    assert "tile 1" in str(e.value)
    bad = dict(b)
    bad["nnzOffset"] = b["nnzOffset"].copy()
    bad["nnzOffset"][0] = 1
    with pytest.raises(hs.HspmmError):
        hs.bitmap_expand(bad)


def test_grouping_equals_oracle(hs, oracle):
    rng = np.random.default_rng(12)
    A = random_csr(rng, 400, 3000, 0.02, 0, 0.2, heavy_rows=(5, 100, 399))
    b = hs.csr_to_bitmap(400, 3000, A["row_ptr"], A["col_idx"], A["values"], 0)
    for min_len in (1, 3, 32, 1000):
        g = hs.bitmap_to_grouped(b, min_len)
        tgl, go, ri, at = oracle.group(b["rowOffset"], b["rowIdx"], min_len)
        assert g["tgl"] == tgl and g["total_groups"] == at.size
        assert np.array_equal(g["groupOffset"], go) and np.array_equal(g["rowIdx"], ri)
        assert np.array_equal(g["atomic"], at)
        assert g["eff_row_windows"] == go.size                      # as the reference sets it (convert.h:267-268)
    empty = hs.csr_to_bitmap(9, 9, np.zeros(10, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.uint16), 0)
    g = hs.bitmap_to_grouped(empty)
    assert g["total_groups"] == 0 and g["groupOffset"].tolist() == [0] and g["tgl"] == 32
