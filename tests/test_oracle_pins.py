"""Pins the CPU oracle (oracle/oracle.c) before anything is compared with it:
golden vectors of the reference's own converter, library routines (numpy,
scipy), closed forms of the reference's micro-tests, exact integer arithmetic
and brute force on small inputs."""
import ctypes
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

from util import IDX_MAX, btcf_to_csr, csr_to_dense64, csr_triples, decode, dtype_name, encode, random_csr

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def gold():
    with open(os.path.join(GOLD, "expected.json")) as f:
        return json.load(f)


# ---------------------------------------------------------------- half <-> float
def test_half_to_float_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_float_to_half_against_numpy(oracle):
    rng = np.random.default_rng(7)
    # every half value, its neighbours' midpoints (ties), and random bit patterns
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = (h[:-1] + h[1:]) / 2
    cases = [h, -h, mids, -mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
             np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
             np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e10, np.inf, -np.inf, 0.0, -0.0,
                       2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 5.96e-8, 6.1e-5]),
             rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)]
    x = np.concatenate([np.asarray(c, np.float32).ravel() for c in cases])
    x = x[~np.isnan(x)]
    got = oracle.f32_to_f16_bits(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert np.isnan(oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(np.array([np.nan], np.float32))))[0]


def test_bfloat16_conversions_against_torch(oracle):
    import torch
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.bf16_bits_to_f32(bits)
    want = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert got.tobytes() == want.tobytes()                      # NaN payloads included
    rng = np.random.default_rng(8)
    f = bits.astype(np.uint32) << 16
    # every bf16 value, the exact midpoints to the next one (ties), their neighbours, random patterns
    cases = [f, f | 0x8000, f | 0x7FFF, f | 0x8001, rng.integers(0, 2 ** 32, 300000, dtype=np.uint64).astype(np.uint32)]
    x = np.concatenate(cases).astype(np.uint32).view(np.float32)
    x = x[~np.isnan(x)]
    got = oracle.f32_to_bf16_bits(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.isnan(oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(np.array([np.nan], np.float32))))[0]
    # the benchmark generator's own conversion agrees as well
    from hopper_spmm_amd import generators as G
    assert np.array_equal(G.bf16_bits(x), want)


# ---------------------------------------------------------------- loader
def test_loader_golden_tiny(oracle):
    g = gold()["tiny"]
    m = oracle.mtx_read(os.path.join(GOLD, g["file"]), "fp16")
    assert (m["rows"], m["cols"], m["nnzs"]) == (g["rows"], g["cols"], g["nnzs"])
    # CSR sorted by (row, col): rows 0,0,1,2,7,7,8,9,9
    assert m["row_ptr"].tolist() == [0, 2, 3, 4, 4, 4, 4, 4, 6, 7, 9]
    assert m["col_idx"].tolist() == [2, 19, 2, 6, 0, 17, 4, 4, 5]
    vals = m["values"].view(np.float16).astype(np.float32).tolist()
    assert vals == [1.5, -2.0, 0.25, 2.0, 4.0, 8.0, -1.0, 3.0, 0.5]


def test_loader_matches_scipy_on_random_files(oracle, tmp_path):
    rng = np.random.default_rng(3)
    for case in range(4):
        rows, cols = int(rng.integers(1, 60)), int(rng.integers(1, 60))
        nnz = int(rng.integers(0, rows * cols // 2 + 1))
        flat = rng.choice(rows * cols, size=nnz, replace=False)
        r, c = flat // cols, flat % cols
        v = rng.normal(size=nnz).astype(np.float32)
        p = tmp_path / ("m%d.mtx" % case)
        with open(p, "w") as f:
            f.write("%%MatrixMarket matrix coordinate real general\n% comment\n")
            f.write("%d %d %d\n" % (rows, cols, nnz))
            for i in range(nnz):
                f.write("%d %d %.9g\n" % (r[i] + 1, c[i] + 1, v[i]))
        for dt in ("fp16", "tf32"):
            m = oracle.mtx_read(str(p), dt)
            ref = sp.coo_matrix((v, (r, c)), shape=(rows, cols)).tocsr()
            ref.sort_indices()
            assert oracle.csr_validate(rows, cols, m["row_ptr"], m["col_idx"]) == 0
            assert np.array_equal(m["row_ptr"], ref.indptr.astype(np.uint32))
            assert np.array_equal(m["col_idx"], ref.indices.astype(np.uint32))
            if dt == "tf32":
                assert np.array_equal(m["values"], ref.data.astype(np.float32))
            else:
                assert np.array_equal(m["values"], ref.data.astype(np.float16).view(np.uint16))


def test_csr_validate_counts_every_kind_of_violation(oracle):
    """orc_csr_validate restates the structural checks of the reference's loader (src/utils/load.h:44-73):
    row_ptr[0] == 0, row_ptr[rows] == nnz, row_ptr never decreasing, every column index below cols.
    Each violation is planted alone and together, and counted."""
    rows, cols = 4, 6
    good_ptr = np.array([0, 2, 2, 5, 6], np.uint32)
    good_idx = np.array([0, 5, 1, 2, 4, 3], np.uint32)
    assert oracle.csr_validate(rows, cols, good_ptr, good_idx) == 0
    # first offset not zero (load.h:44-47); the offsets stay ascending and end at nnz
    assert oracle.csr_validate(rows, cols, np.array([1, 2, 2, 5, 6], np.uint32), good_idx) == 1
    # last offset differs from the number of entries (load.h:49-53)
    assert oracle.csr_validate(rows, cols, np.array([0, 2, 2, 5, 5], np.uint32), good_idx) == 1
    # offsets that decrease, once and twice (load.h:56-62)
    assert oracle.csr_validate(rows, cols, np.array([0, 3, 2, 5, 6], np.uint32), good_idx) == 1
    assert oracle.csr_validate(rows, cols, np.array([0, 3, 2, 1, 6], np.uint32), good_idx) == 2
    # column indices outside the matrix, one and three of them (load.h:66-73); cols - 1 is the last valid one
    bad_idx = good_idx.copy(); bad_idx[1] = cols
    assert oracle.csr_validate(rows, cols, good_ptr, bad_idx) == 1
    bad_idx[[0, 4]] = [cols + 7, 0xFFFFFFFF]
    assert oracle.csr_validate(rows, cols, good_ptr, bad_idx) == 3
    # everything at once: 1 (first offset) + 1 (last offset) + 1 (decrease) + 3 (columns)
    assert oracle.csr_validate(rows, cols, np.array([1, 3, 2, 5, 7], np.uint32), bad_idx) == 6
    # an empty matrix is valid
    assert oracle.csr_validate(0, 0, np.array([0], np.uint32), np.zeros(0, np.uint32)) == 0


def test_loader_failure_paths(oracle, tmp_path):
    with pytest.raises(OSError):
        oracle.mtx_read(str(tmp_path / "missing.mtx"), "fp16")          # load.h:176-180
    bad = tmp_path / "bad.mtx"
    bad.write_text("%%MatrixMarket\nnot a size line\n")
    with pytest.raises(ValueError):
        oracle.mtx_read(str(bad), "fp16")                                 # load.h:190-194
    # fewer entries than declared: warning path shrinks nnz (load.h:234-238);
    # a line that is not three fields is skipped (load.h:219)
    short = tmp_path / "short.mtx"
    short.write_text("%%MatrixMarket\n3 3 5\n1 1 1.0\n2 2\n3 3 2.5\n")
    m = oracle.mtx_read(str(short), "tf32")
    assert m["declared_nnz"] == 5 and m["nnzs"] == 2
    assert m["col_idx"].tolist() == [0, 2] and m["values"].tolist() == [1.0, 2.5]
    # pattern file (two fields per line) yields no entries
    pat = tmp_path / "pat.mtx"
    pat.write_text("%%MatrixMarket matrix coordinate pattern general\n2 2 2\n1 1\n2 2\n")
    assert oracle.mtx_read(str(pat), "fp16")["nnzs"] == 0


# ---------------------------------------------------------------- converter
def _check_golden_btcf(b, g):
    assert b["total_row_windows"] == g["total_row_windows"]
    assert b["eff_row_windows"] == g["eff_row_windows"]
    assert b["total_tiles"] == g["total_tiles"]
    assert b["data"].size == g["data_size"]
    assert b["rowOffset"].tolist() == g["rowOffset"]
    assert b["rowIdx"].tolist() == g["rowIdx"]
    assert b["tcA2B"].tolist() == g["tcA2B"]
    if "tile_nonzeros" in g:
        cw = b["cw"]
        want = np.zeros((g["total_tiles"], 8, cw), np.float32)
        for t, r, k, v in g["tile_nonzeros"]:
            want[t, r, k] = v
        got = b["data"].view(np.float16).astype(np.float32) if b["dtype"] == "fp16" or b["dtype"] == 0 else b["data"]
        assert np.array_equal(got.reshape(want.shape), want)


def test_converter_golden_vectors(oracle):
    G = gold()
    for name in ("tiny", "gap"):
        g = G[name]
        m = oracle.mtx_read(os.path.join(GOLD, g["file"]), g["dtype"])
        b = oracle.csr_to_btcf(m["rows"], m["cols"], m["row_ptr"], m["col_idx"], m["values"], g["dtype"])
        _check_golden_btcf(b, g)


def _format_invariants(b, A):
    W, T, cw = b["eff_row_windows"], b["total_tiles"], b["cw"]
    ro, ri = b["rowOffset"].astype(np.int64), b["rowIdx"].astype(np.int64)
    assert ro[0] == 0 and ro[-1] == T and np.all(np.diff(ro) > 0)
    assert np.all(ri % 8 == 0) and np.all(np.diff(ri) > 0)
    a2b = b["tcA2B"].reshape(T, cw)
    for w in range(W):
        ids = a2b[ro[w]:ro[w + 1]].ravel()
        real = ids[ids != IDX_MAX]
        assert np.all(np.diff(real.astype(np.int64)) > 0)            # strictly ascending
        assert np.all(ids[real.size:] == IDX_MAX)                    # padding only at the end
        assert ids.size - real.size < cw                             # ... and only in the last tile
        rp = A["row_ptr"]
        r0, r1 = ri[w], min(ri[w] + 8, A["rows"])
        assert np.array_equal(real, np.unique(A["col_idx"][rp[r0]:rp[r1]]))
    # windows that are not listed hold no entry
    listed = set(ri.tolist())
    for r0 in range(0, A["rows"], 8):
        n = int(A["row_ptr"][min(r0 + 8, A["rows"])]) - int(A["row_ptr"][r0])
        assert (n > 0) == (r0 in listed)


@pytest.mark.parametrize("dtype", [0, 1])
def test_converter_round_trip_and_invariants(oracle, dtype):
    rng = np.random.default_rng(11 + dtype)
    for rows, cols, dens, erp in [(1, 1, 1.0, 0), (7, 5, 0.5, 0), (8, 40, 0.3, 0.2), (27, 100, 0.1, 0.5),
                                  (64, 33, 0.4, 0.0), (100, 300, 0.02, 0.6)]:
        A = random_csr(rng, rows, cols, dens, dtype, erp)
        b = oracle.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], "fp16" if dtype == 0 else "tf32")
        _format_invariants(b, A)
        got = btcf_to_csr(b)
        want = [(r, c, v) for r, c, v in csr_triples(A) if v != 0]
        assert [(r, c) for r, c, _ in got] == [(r, c) for r, c, _ in want]
        assert all(gv == wv for (_, _, gv), (_, _, wv) in zip(got, want))


def test_converter_brute_force_dense(oracle):
    """Every 0/1 pattern of a 9 x 3 matrix is too many; take all 2^9 patterns of a
    3 x 3 corner inside a 9 x 20 matrix plus fixed far columns and compare with a
    direct construction from the definition."""
    for pat in range(0, 512, 7):
        D = np.zeros((9, 20), np.float32)
        for bit in range(9):
            if pat >> bit & 1:
                D[bit // 3 * 4, (bit % 3) * 9] = bit + 1
        D[8, 19] = 42
        rp = np.zeros(10, np.uint32)
        ci, vv = [], []
        for r in range(9):
            nz = np.nonzero(D[r])[0]
            ci += nz.tolist(); vv += D[r, nz].tolist()
            rp[r + 1] = len(ci)
        b = oracle.csr_to_btcf(9, 20, rp, np.array(ci, np.uint32), np.array(vv, np.float32), "tf32")
        # definition: per 8-row window, sorted distinct columns, 8 per tile
        exp_ids, exp_tiles = [], []
        for r0 in (0, 8):
            blk = D[r0:r0 + 8]
            cols = np.nonzero(blk.any(axis=0))[0]
            if cols.size == 0:
                continue
            padded = list(cols) + [IDX_MAX] * (-cols.size % 8)
            exp_ids += padded
            for t in range(len(padded) // 8):
                tile = np.zeros((8, 8), np.float32)
                for k in range(8):
                    c = padded[t * 8 + k]
                    if c != IDX_MAX:
                        tile[:blk.shape[0], k] = blk[:, c]
                exp_tiles.append(tile)
        assert b["tcA2B"].tolist() == exp_ids
        assert np.array_equal(b["data"].reshape(-1, 8, 8), np.array(exp_tiles))


# ---------------------------------------------------------------- bitmap tiles and groups
def _expand_bitmap(b):
    """Definition of the bitmap format, in numpy: the k-th stored entry of a tile
    sits where its k-th set bit is."""
    cw, T = b["cw"], b["total_tiles"]
    words = b["tcBit"].size // max(T, 1) if T else 1
    dense = np.zeros((T, 8 * cw), b["data"].dtype)
    for t in range(T):
        bits = 0
        for k in range(words):
            bits |= int(b["tcBit"][t * words + k]) << (64 * k)
        pos = [i for i in range(8 * cw) if bits >> i & 1]
        seg = b["data"][b["nnzOffset"][t]:b["nnzOffset"][t + 1]]
        assert len(pos) == seg.size
        dense[t, pos] = seg
    return dense.ravel()


def test_bitmap_golden_vector(oracle):
    g = gold()["tiny"]
    m = oracle.mtx_read(os.path.join(GOLD, g["file"]), "fp16")
    b = oracle.csr_to_bitmap(m["rows"], m["cols"], m["row_ptr"], m["col_idx"], m["values"], "fp16", as_reference=True)
    assert b["nnzOffset"].tolist() == g["bitmap"]["nnzOffset"]
    assert b["data"].view(np.float16).astype(np.float32).tolist() == g["bitmap"]["data"]
    assert [int(x) for x in b["tcBit"]] == [int(x, 16) for x in g["bitmap"]["tcBit_as_reference"]]
    assert b["rowOffset"].tolist() == g["rowOffset"] and b["tcA2B"].tolist() == g["tcA2B"]
    assert b["rowIdx"].tolist() == g["rowIdx"]
    # the per-tile layout holds the same bits, two words to a tile
    c = oracle.csr_to_bitmap(m["rows"], m["cols"], m["row_ptr"], m["col_idx"], m["values"], "fp16")
    want = np.zeros((2, 128), bool)
    for t, r, k, _ in g["tile_nonzeros"]:
        want[t, r * 16 + k] = True
    got = np.array([[int(c["tcBit"][2 * t + i // 64]) >> (i % 64) & 1 for i in range(128)] for t in range(2)], bool)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_bitmap_expands_to_the_uncompressed_tiles(oracle, dtype):
    rng = np.random.default_rng(300 + dtype)
    name = dtype_name(dtype)
    for rows, cols, dens, erp in [(1, 1, 1.0, 0), (7, 5, 0.5, 0), (8, 40, 0.9, 0.0), (27, 100, 0.1, 0.5),
                                  (64, 33, 0.4, 0.0), (100, 300, 0.02, 0.6)]:
        A = random_csr(rng, rows, cols, dens, dtype, erp)
        A["values"][A["values"] == 0] = encode(np.float32(0.5), dtype)    # stored zeros would hide a misplaced entry
        for tr in (False, True):
            b = oracle.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], name, transpose=tr)
            d = oracle.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], name, transpose=tr)
            for k in ("rowOffset", "tcA2B", "rowIdx"):
                assert np.array_equal(b[k], d[k])
            assert b["nnzOffset"][0] == 0 and b["nnzOffset"][-1] == A["nnzs"] and b["data"].size == A["nnzs"]
            assert np.array_equal(_expand_bitmap(b).view(np.uint8), d["data"].view(np.uint8))
            # as-reference indexing: 8 x 8 tiles are unaffected; for 8 x 16 tiles word w is the
            # low word of tile w or-ed with the high word of tile w - 1
            r = oracle.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], name, transpose=tr,
                                     as_reference=True)
            if dtype == 1:
                assert np.array_equal(r["tcBit"], b["tcBit"])
            else:
                T = b["total_tiles"]
                lo, hi = b["tcBit"][0::2], b["tcBit"][1::2]
                want = np.zeros(2 * T, np.uint64)
                want[:T] |= lo
                want[1:T + 1] |= hi
                assert np.array_equal(r["tcBit"], want)


def test_grouping_hand_computed_and_closed_form(oracle):
    # tiles per window 5, 65, 1, 129: mean 50 -> tgl 50; 65 -> 2 groups 33 apart; 129 -> 3 groups 43 apart
    tgl, go, ri, at = oracle.group(np.array([0, 5, 70, 71, 200]), np.array([0, 8, 24, 32]))
    assert tgl == 50
    assert go.tolist() == [0, 5, 38, 70, 71, 114, 157, 200]
    assert ri.tolist() == [0, 8, 8, 24, 32, 32, 32]
    assert at.tolist() == [0, 1, 1, 0, 1, 1, 1]
    # mean below the floor of 32 tiles: tgl = 32
    tgl, go, ri, at = oracle.group(np.array([0, 3, 36]), np.array([8, 16]))
    assert tgl == 32 and go.tolist() == [0, 3, 20, 36] and at.tolist() == [0, 1, 1] and ri.tolist() == [8, 16, 16]
    # no window at all
    tgl, go, ri, at = oracle.group(np.array([0]), np.zeros(0, np.uint32))
    assert tgl == 32 and go.tolist() == [0] and ri.size == 0
    rng = np.random.default_rng(5)
    for min_len in (1, 4, 32):
        n = rng.integers(1, 400, 60)
        ro = np.concatenate([[0], np.cumsum(n)])
        ri_in = np.arange(60) * 8
        tgl, go, ri, at = oracle.group(ro, ri_in, min_len)
        assert tgl == max(int(n.sum() / 60), min_len)
        g = 0
        for w in range(60):
            k = -(-int(n[w]) // tgl)
            step = -(-int(n[w]) // k)
            assert go[g:g + k].tolist() == [int(ro[w]) + step * j for j in range(k)]
            assert np.all(ri[g:g + k] == ri_in[w]) and np.all(at[g:g + k] == (k > 1))
            # every group holds at least one and at most tgl tiles, together exactly the window
            ends = go[g + 1:g + k + 1].astype(np.int64)
            sizes = ends - go[g:g + k]
            assert ends[-1] == ro[w + 1] and np.all(sizes >= 1) and np.all(sizes <= tgl)
            g += k
        assert g == at.size and go[-1] == ro[-1]


def test_converter_duplicate_entries_last_one_wins(oracle):
    # convert.h:215 assigns, it does not add: of two stored entries at one position
    # the later one (in CSR order) stays
    rp = np.array([0, 3], np.uint32)
    ci = np.array([4, 4, 9], np.uint32)
    vv = np.array([1.0, 2.0, 3.0], np.float32)
    b = oracle.csr_to_btcf(1, 10, rp, ci, vv, "tf32")
    assert b["tcA2B"].tolist()[:2] == [4, 9] and b["data"][0] == 2.0 and b["data"][1] == 3.0


def test_converter_transposed_tile_order(oracle):
    rng = np.random.default_rng(5)
    A = random_csr(rng, 20, 50, 0.3, 0)
    b0 = oracle.csr_to_btcf(20, 50, A["row_ptr"], A["col_idx"], A["values"], "fp16")
    b1 = oracle.csr_to_btcf(20, 50, A["row_ptr"], A["col_idx"], A["values"], "fp16", transpose=True)
    assert np.array_equal(b0["tcA2B"], b1["tcA2B"])
    t0 = b0["data"].reshape(-1, 8, 16)
    t1 = b1["data"].reshape(-1, 16, 8)
    assert np.array_equal(t0, t1.transpose(0, 2, 1))                 # convert.h:207-212


# ---------------------------------------------------------------- SpMM arithmetic
def test_spmm_exact_integer_case(oracle):
    """Small integers: every product and partial sum is exact in fp32 and the result
    is exact in fp16, so the oracle must equal the integer matrix product bit for
    bit; a transposed B, a dropped term or a wrong index cannot survive this."""
    rng = np.random.default_rng(21)
    rows, cols, N = 37, 29, 12
    D = rng.integers(-3, 4, (rows, cols)) * (rng.random((rows, cols)) < 0.3)
    Bm = rng.integers(-4, 5, (cols, N))
    want = D @ Bm
    rp = np.zeros(rows + 1, np.uint32)
    ci, vv = [], []
    for r in range(rows):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    ci = np.array(ci, np.uint32)
    v16 = np.array(vv, np.float32).astype(np.float16).view(np.uint16)
    B16 = Bm.astype(np.float16).view(np.uint16)
    C = oracle.spmm_csr_f16(rows, N, rp, ci, v16, B16)
    assert np.array_equal(C.view(np.float16).astype(np.int64), want)
    C32 = oracle.spmm_csr_f32(rows, N, rp, ci, np.array(vv, np.float32), Bm.astype(np.float32))
    assert np.array_equal(C32.astype(np.int64), want)
    for dt, vals, Bx in (("fp16", v16, B16), ("tf32", np.array(vv, np.float32), Bm.astype(np.float32))):
        b = oracle.csr_to_btcf(rows, cols, rp, ci, vals, dt)
        Ct = oracle.spmm_btcf(b, Bx, N)
        got = Ct.view(np.float16).astype(np.int64) if dt == "fp16" else Ct.astype(np.int64)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_spmm_against_dense_float64(oracle, dtype):
    rng = np.random.default_rng(31 + dtype)
    rows, cols, N = 50, 70, 24
    A = random_csr(rng, rows, cols, 0.2, dtype, 0.2)
    Bf = rng.normal(size=(cols, N)).astype(np.float32)
    B = encode(Bf, dtype)
    B64 = decode(B, dtype)
    exact = csr_to_dense64(A) @ B64
    mag = np.abs(csr_to_dense64(A)) @ np.abs(B64)
    if dtype == 0:
        C, absdot = oracle.spmm_csr_f16(rows, N, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)
        got = C.view(np.float16).astype(np.float64)
        # one fp16 rounding of an fp32 sum: half an ulp of the result plus fp32 noise
        assert np.all(np.abs(got - exact) <= np.abs(exact) * 2.0 ** -11 + mag * 1e-6 + 1e-7)
    elif dtype == 2:
        C, absdot = oracle.spmm_csr_bf16(rows, N, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)
        got = decode(C, 2)
        # one bf16 rounding (8 significant bits: half an ulp is at most 2^-8 relative) of an fp32 sum
        assert np.all(np.abs(got - exact) <= np.abs(exact) * 2.0 ** -8 + mag * 1e-6 + 1e-30)
    else:
        C, absdot = oracle.spmm_csr_f32(rows, N, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)
        assert np.all(np.abs(C - exact) <= mag * 1e-6)
    assert np.allclose(absdot, mag, rtol=1e-5, atol=1e-7)
    # tile order and CSR order agree to reassociation error (identical here: both go k ascending)
    b = oracle.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype_name(dtype))
    Ct = oracle.spmm_btcf(b, B, N)
    if dtype != 1:
        assert np.array_equal(Ct, C)
    else:
        assert np.allclose(Ct, C, rtol=1e-6, atol=1e-6)


def test_spmm_tf32_truncation_option(oracle):
    rng = np.random.default_rng(2)
    A = random_csr(rng, 16, 16, 0.5, 1)
    B = rng.normal(size=(16, 8)).astype(np.float32)
    Ct = oracle.spmm_csr_f32(16, 8, A["row_ptr"], A["col_idx"], A["values"], B, trunc_tf32=True)
    mask = np.uint32(0xFFFFE000)
    At = A.copy(); At["values"] = (A["values"].view(np.uint32) & mask).view(np.float32)
    Bt = (B.view(np.uint32) & mask).view(np.float32)
    want = csr_to_dense64(At) @ Bt.astype(np.float64)
    assert np.allclose(Ct, want, rtol=1e-5, atol=1e-6)
    full, mag = oracle.spmm_csr_f32(16, 8, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)
    # truncating both inputs to 10 mantissa bits moves each product by < 2^-9 of its size
    assert np.all(np.abs(Ct - full) <= mag * 2.0 ** -9)
    assert not np.array_equal(Ct, full)


# ---------------------------------------------------------------- micro-test known answers
def test_tile_mma_fp16_known_answer(oracle):
    # reference src/test_fp16.cu:407-415: A[i] = half(i + 1) (64 x 16), B = 1 (8 x 16)
    A = (np.arange(64 * 16) + 1).astype(np.float32).astype(np.float16)
    B = np.ones(8 * 16, np.float16)
    C = oracle.tile_mma_f16(A.view(np.uint16), B.view(np.uint16), 64, 8, 16)
    # all entries are <= 1024, exact in half: sum_{k=1..16} (16 i + k) = 256 i + 136
    i = np.arange(64)
    assert np.array_equal(C, np.repeat((256 * i + 136)[:, None], 8, axis=1).astype(np.float32))
    want = A.astype(np.float64).reshape(64, 16).sum(axis=1)          # rounded halves, exact sum
    assert np.array_equal(C, np.repeat(want[:, None], 8, axis=1).astype(np.float32))


def test_tile_mma_tf32_known_answer(oracle):
    # reference test/02.tma_and_wgmma/tma_wgmma.cu:340-348: A[i] = i + 1 (64 x 8), B[i] = 1 + 0.01 i (8 x 8)
    A = (np.arange(64 * 8) + 1).astype(np.float32)
    B = (1.0 + np.arange(64, dtype=np.float32) * np.float32(0.01)).astype(np.float32)
    C = oracle.tile_mma_f32(A, B, 64, 8, 8)
    i, j, k = np.meshgrid(np.arange(64), np.arange(8), np.arange(8), indexing="ij")
    want = ((8 * i + k + 1) * B.astype(np.float64)[8 * j + k]).sum(axis=2)
    assert np.allclose(C, want, rtol=1e-6)
    assert oracle.verdict_rel(want.astype(np.float32), C, 1e-2) == 0
    # a transposed B operand is a different answer
    assert not np.allclose(oracle.tile_mma_f32(A, B.reshape(8, 8).T.copy().ravel(), 64, 8, 8), want, rtol=1e-3)


def test_tile_accumulate_with_reference_inputs(oracle):
    # reference test/03.warp_specialized/main.cu:235-241: srand(42), rand()/RAND_MAX,
    # A 64 x (8 T) row-major, B 8 x (8 T) K-major; check of utils.h:26-97
    libc = ctypes.CDLL("libc.so.6")
    libc.rand.restype = ctypes.c_int
    T = 5
    libc.srand(42)
    A = np.array([libc.rand() for _ in range(64 * 8 * T)], np.float32) / np.float32(2147483647)
    B = np.array([libc.rand() for _ in range(8 * T * 8)], np.float32) / np.float32(2147483647)
    C = oracle.tile_accum_f32(A, B, 64, 8, 8, T)
    want = A.astype(np.float64).reshape(64, 8 * T) @ B.astype(np.float64).reshape(8, 8 * T).T
    assert np.allclose(C, want, rtol=1e-5)
    assert oracle.verdict_rel_abs(C, want.astype(np.float32), 1e-2) == 0


def test_verdict_forms(oracle):
    e = np.array([1.0, 100.0, 0.0, 1e-7, -2.0], np.float32)
    a = np.array([1.009, 102.0, 0.0, 2e-6, -2.03], np.float32)
    # form 1 (test_fp16.cu:302-309): |e-a| / (|e| + 1e-8) > tol -> entries 1, 3, 4 fail
    assert oracle.verdict_rel(e, a, 1e-2) == 3
    # form 2 (tf32.cu:46-70): relative when |ref| > 1e-6 else absolute 1e-5 -> entries 1 and 4 fail
    assert oracle.verdict_rel_abs(a, e, 1e-2) == 2
    assert oracle.verdict_rel(e, e, 1e-2) == 0 and oracle.verdict_rel_abs(e, e, 1e-2) == 0
