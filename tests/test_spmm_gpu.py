"""Parity of the HIP operator (through the C ABI of libhspmm.so) with the CPU
oracle on the same seeded inputs.  Needs a real MI355X: run with -m gpu.

Tolerances (from the task's statement of parity):
  fp16 path : |gpu - ref| <= 1e-2 * |ref| + 1e-5 * sum_k |a_k b_k|
  tf32 path : |gpu - ref| <= 1e-3 * |ref| + 1e-5 * sum_k |a_k b_k|
  bf16 path : the fp16 bound (one bf16 rounding is 2^-9 relative)
The second term only matters where a sum cancels to (almost) nothing; it is the
size of fp32 reassociation noise.  Index handling is checked bit-exactly through
cases whose arithmetic is exact (small integers) and through the format tests.
"""
import os

import numpy as np
import pytest

from util import built_depth, csr_to_dense64, decode, encode, half_ulp_distance, random_csr

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DT = {0: "fp16", 1: "tf32", 2: "bf16"}


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


def gpu_spmm(torch, hs, btcf, B, N, plan=None, poison=True, offsets=None):
    """C = A*B on the device through hspmm_run; B, C as numpy (uint16 bits / float32).
    offsets = (bytes, bytes): B and C start that far (multiples of the element size, < 64) into their
    allocations, and the bytes around C must come back untouched."""
    own = plan is None
    if own:
        plan = hs.Plan(btcf)
    dt = btcf["dtype"]
    rows = btcf["rows"]
    stream = torch.cuda.current_stream().cuda_stream
    if offsets is not None:
        off_b, off_c = offsets
        host_b = np.ascontiguousarray(B, np.float32 if dt == 1 else np.uint16)
        bytes_b = torch.from_numpy(host_b.view(np.uint8).reshape(-1))
        raw_b = torch.zeros(bytes_b.numel() + 128, dtype=torch.uint8, device="cuda")
        raw_b[off_b:off_b + bytes_b.numel()].copy_(bytes_b)
        size_c = rows * N * host_b.itemsize
        raw_c = torch.full((size_c + 256,), 0xA5, dtype=torch.uint8, device="cuda")     # (fp32: a NaN pattern too)
        plan.run(raw_b.data_ptr() + off_b, raw_c.data_ptr() + 64 + off_c, N, stream)
        torch.cuda.synchronize()
        host_c = raw_c.cpu().numpy()
        if own:
            plan.close()
        assert (host_c[:64 + off_c] == 0xA5).all() and (host_c[64 + off_c + size_c:] == 0xA5).all(), "bytes next to C written"
        return host_c[64 + off_c:64 + off_c + size_c].copy().view(host_b.dtype).reshape(rows, N)
    if dt != 1:
        dB = torch.from_numpy(np.ascontiguousarray(B, np.uint16).view(np.int16)).cuda()
        dC = torch.empty((rows, N), dtype=torch.int16, device="cuda")
        if poison:
            dC.fill_(0x7E01)                     # a NaN pattern: unwritten elements show up
    else:
        dB = torch.from_numpy(np.ascontiguousarray(B, np.float32)).cuda()
        dC = torch.empty((rows, N), dtype=torch.float32, device="cuda")
        if poison:
            dC.fill_(float("nan"))
    plan.run(dB.data_ptr(), dC.data_ptr(), N, stream)
    torch.cuda.synchronize()
    out = dC.cpu().numpy()
    if own:
        plan.close()
    return out.view(np.uint16) if dt != 1 else out


def oracle_spmm(oracle, A, B, N):
    if A["dtype"] == 2:
        return oracle.spmm_csr_bf16(A["rows"], N, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)
    if A["dtype"] == 0:
        return oracle.spmm_csr_f16(A["rows"], N, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)
    return oracle.spmm_csr_f32(A["rows"], N, A["row_ptr"], A["col_idx"], A["values"], B, want_absdot=True)


def assert_parity(got, ref, absdot, dtype, what="", tight=True):
    """fp16 / bf16: 1e-2 relative; fp32-storage ("tf32") variant: 1e-3 relative.  Where the sum
    cancels, an absolute term in units of sum |a||b|: 1e-5 for fp32 accumulation of exact products.
    The tf32 variant's LDS-staging kernels multiply bf16 hi + lo parts in three products (unless the
    kernel mode guarantees fp32 products).  The product they leave out, a_lo b_lo, has the sign of a b
    and at most 2^-14 of its size (2^-16 on average), so every output must lie within 2^-14 sum |a||b|
    more - the hard bound, reached only by factors with every low mantissa bit set - and all but one in
    10^5 of them (one of an array smaller than that) within 2^-16 sum |a||b|: measured on normal entries
    against fp64 the worst is 2^-17.3 sum |a||b|, and of 10^9 outputs of random inputs five lay beyond
    2^-16 (tf32 itself: 2^-10)."""
    import hopper_spmm_amd
    parts = dtype == 1 and hopper_spmm_amd.get_kernel_mode() not in (1, 2, 3, 5)
    if dtype != 1:
        g, r, rel, absolute = decode(got, dtype), decode(ref, dtype), 1e-2, 1e-5
    else:
        g, r, rel = got.astype(np.float64), ref.astype(np.float64), 1e-3
        absolute = 1e-5 + 2.0 ** -14 if parts else 1e-5
    assert not np.isnan(g).any(), what + ": unwritten or NaN output"
    err = np.abs(g - r)
    bound = rel * np.abs(r) + absolute * absdot.astype(np.float64)
    bad = err > bound
    assert not bad.any(), "%s: %d of %d outputs outside tolerance, worst %g at %s" % (
        what, int(bad.sum()), bad.size, float((err - bound).max()), np.unravel_index(np.argmax(err - bound), err.shape))
    if parts:
        beyond = err > rel * np.abs(r) + (1e-5 + 2.0 ** -16) * absdot.astype(np.float64)
        assert int(beyond.sum()) <= max(1, beyond.size // 100000), "%s: %d of %d outputs beyond 2^-16 sum |a||b|" % (
            what, int(beyond.sum()), beyond.size)
    if tight and dtype != 1 and got.size:
        # far tighter in practice (except for long, cancelling sums): one rounding of nearly identical fp32 sums
        ulp = half_ulp_distance(got, ref)
        assert (ulp <= 1).mean() > 0.999, what + ": too many outputs differ by more than one half ulp"


def make_b(rng, cols, N, dtype):
    x = rng.normal(size=(cols, N)).astype(np.float32)
    return encode(x, dtype)


def convert(hs, A):
    return hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], A["dtype"])


# ------------------------------------------------------------------ golden files
def test_golden_files_end_to_end(torch_cuda, hs, oracle):
    rng = np.random.default_rng(1)
    for name, dt in (("tiny.mtx", 0), ("gap.mtx", 1)):
        A = hs.mtx_load(os.path.join(GOLD, name), dt)
        A["dtype"] = dt
        b = convert(hs, A)
        for N in (1, 2, 3, 8, 16, 40, 64, 128):
            B = make_b(rng, A["cols"], N, dt)
            got = gpu_spmm(torch_cuda, hs, b, B, N)
            ref, mag = oracle_spmm(oracle, A, B, N)
            assert_parity(got, ref, mag, dt, "%s N=%d" % (name, N))
            # gap.mtx: rows 8..23 lie in no effective window and the last window has
            # three real rows; all of that must come out as exact zeros
            dense = csr_to_dense64(A)
            empty = ~dense.any(axis=1)
            assert not got[empty].any()


# ------------------------------------------------------------------ exact arithmetic: bit-exact
@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_exact_integer_inputs_are_bit_exact(torch_cuda, hs, oracle, dtype, mode):
    rng = np.random.default_rng(40 + dtype)
    rows, cols = 203, 310
    D = rng.integers(-3, 4, (rows, cols)) * (rng.random((rows, cols)) < 0.15)
    D[40:56] = 0                                    # two empty windows in the middle
    rp = np.zeros(rows + 1, np.uint32)
    ci, vv = [], []
    for r in range(rows):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    vals = np.array(vv, np.float32)
    A = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32),
             values=encode(vals, dtype))
    hs.set_kernel_mode(mode)
    try:
        b = convert(hs, A)
        for N in (4, 32, 64, 128, 160):
            Bm = rng.integers(-4, 5, (cols, N))
            B = encode(Bm, dtype)
            got = gpu_spmm(torch_cuda, hs, b, B, N)
            # the sums are exact in fp32, so the output is the one rounding of the
            # exact integer result to the storage type
            want = encode(D @ Bm, dtype)
            assert np.array_equal(got, want), "mode %d N %d" % (mode, N)
            if dtype != 2:
                assert np.array_equal(decode(got, dtype).astype(np.int64), D @ Bm)
    finally:
        hs.set_kernel_mode(0)


# ------------------------------------------------------------------ shapes, tails, splits
SHAPES = [
    # rows, cols, density, empty-row probability, heavy rows
    (1, 1, 1.0, 0.0, ()),
    (7, 33, 0.4, 0.0, ()),
    (8, 16, 1.0, 0.0, ()),
    (27, 100, 0.1, 0.5, ()),
    (130, 257, 0.05, 0.3, ()),
    (300, 3000, 0.004, 0.2, (5, 100, 101, 299)),    # heavy windows: cut across ranges
    (1000, 700, 0.01, 0.6, (512,)),
]


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("shape", SHAPES)
def test_random_shapes_and_feature_dims(torch_cuda, hs, oracle, dtype, shape):
    rows, cols, dens, erp, heavy = shape
    rng = np.random.default_rng(hash((rows, cols, dtype)) & 0xFFFF)
    A = random_csr(rng, rows, cols, dens, dtype, erp, heavy)
    b = convert(hs, A)
    # many ranges, so that heavy windows are split and partial sums are exercised
    hs.configure(producer_warp_group_num=16)
    try:
        plan = hs.Plan(b)
    finally:
        hs.configure()
    if heavy and cols >= 3000:
        assert plan.info()["n_split_windows"] > 0
    # (10, 30, 100, 130, 250 and, for fp32 storage, 5, 7, 127: feature dimensions that no wide load divides run as two
    # launches, the features up to the last multiple of 8 resp. 4 and the few behind it)
    for N in (1, 2, 5, 6, 7, 8, 10, 16, 24, 30, 32, 64, 72, 96, 100, 127, 128, 130, 200, 250, 256, 384):
        B = make_b(rng, cols, N, dtype)
        got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(got, ref, mag, dtype, "shape %s N=%d" % (shape[:2], N), tight=got.size >= 10000)
    plan.close()


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("mode", [1, 2, 3])
@pytest.mark.parametrize("stages", [1, 2, 3, 4, 6, 8])
def test_kernel_variants_agree_with_oracle(torch_cuda, hs, oracle, dtype, mode, stages):
    if stages not in (2, 3, 4) and not hs.has_experimental():
        pytest.skip("prefetch depth %d exists in libraries built with EXPERIMENTAL=1 only" % stages)
    rng = np.random.default_rng(77)
    A = random_csr(rng, 260, 2000, 0.01, dtype, 0.2, (17, 130))
    b = convert(hs, A)
    hs.set_kernel_mode(mode)
    hs.configure(buffer_stage=stages, consumer_warp_num=1 + stages % 4, producer_warp_group_num=8)
    try:
        plan = hs.Plan(b)
        for N in (32, 64, 128, 512):
            B = make_b(rng, 2000, N, dtype)
            got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
            ref, mag = oracle_spmm(oracle, A, B, N)
            assert_parity(got, ref, mag, dtype, "mode %d stages %d N=%d" % (mode, stages, N))
        plan.close()
    finally:
        hs.set_kernel_mode(0)
        hs.configure()


def _block_matrix(rng, rows, cols, brows, bcols, keep, dtype, break_some=False):
    """Nonzeros clustered in brows x bcols blocks; optionally a few extra entries that
    make some window pairs differ."""
    D = np.zeros((rows, cols), np.float32)
    for bi in range(0, rows, brows):
        for bj in range(0, cols, bcols):
            if rng.random() < keep:
                blk = rng.uniform(-1, 1, (min(brows, rows - bi), min(bcols, cols - bj))).astype(np.float32)
                blk[blk == 0] = 0.5
                D[bi:bi + brows, bj:bj + bcols] = blk
    if break_some:
        for _ in range(rows // 40):
            D[rng.integers(0, rows), rng.integers(0, cols)] = 0.25
    rp = np.zeros(rows + 1, np.uint32)
    ci, vv = [], []
    for r in range(rows):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    vals = np.array(vv, np.float32)
    return dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32),
                values=encode(vals, dtype))


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("case", ["blocks16", "blocks32", "mixed", "ragged"])
def test_windows_with_one_column_list_share_their_gather(torch_cuda, hs, oracle, dtype, case):
    rng = np.random.default_rng(60 + dtype)
    if case == "blocks16":
        A = _block_matrix(rng, 256, 1200, 16, 16, 0.5, dtype)
    elif case == "blocks32":
        A = _block_matrix(rng, 288, 900, 32, 24, 0.4, dtype)
    elif case == "mixed":
        A = _block_matrix(rng, 400, 800, 16, 16, 0.5, dtype, break_some=True)
    else:
        A = _block_matrix(rng, 203, 500, 16, 8, 0.6, dtype)          # rows % 16 != 0: last pair is ragged
    b = convert(hs, A)
    for pairing, stages in ((0, 0), (2, 0), (2, 1 if hs.has_experimental() else 3), (2, 4), (1, 0)):
        hs.set_window_pairing(pairing)
        hs.configure(buffer_stage=stages, producer_warp_group_num=16)
        try:
            plan = hs.Plan(b)
        finally:
            hs.set_window_pairing(0)
            hs.configure()
        info = plan.info()
        if pairing == 1:
            assert info["n_paired_units"] == 0 and info["n_units"] == info["eff_row_windows"]
        elif case != "mixed" or pairing == 2:
            assert info["n_paired_units"] > 0
            assert info["n_units"] + info["n_paired_units"] == info["eff_row_windows"]
        for N in (8, 32, 64, 128, 256):
            B = make_b(rng, A["cols"], N, dtype)
            got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
            ref, mag = oracle_spmm(oracle, A, B, N)
            assert_parity(got, ref, mag, dtype, "%s pairing %d stages %d N=%d" % (case, pairing, stages, N))
        plan.close()


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_plans_from_bitmap_and_grouped_formats(torch_cuda, hs, oracle, dtype):
    """The compressed and the grouped format describe the same matrix: their plans
    give bit for bit what the plan of the uncompressed tiles gives, and that agrees
    with the oracle."""
    rng = np.random.default_rng(90 + dtype)
    for rows, cols, dens, erp, heavy in [(27, 100, 0.1, 0.5, ()), (300, 3000, 0.004, 0.2, (5, 100, 101, 299)),
                                         (1000, 700, 0.01, 0.6, (512,))]:
        A = random_csr(rng, rows, cols, dens, dtype, erp, heavy)
        plain = convert(hs, A)
        bitmap = hs.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype)
        assert bitmap["data"].size == A["nnzs"] < plain["data"].size
        grouped = hs.bitmap_to_grouped(bitmap, min_len=4)
        if heavy:
            assert grouped["atomic"].any()
        for N in (8, 64, 136):
            B = make_b(rng, cols, N, dtype)
            want = gpu_spmm(torch_cuda, hs, plain, B, N)
            ref, mag = oracle_spmm(oracle, A, B, N)
            assert_parity(want, ref, mag, dtype, "plain %dx%d N=%d" % (rows, cols, N))
            for name, fmt in (("bitmap", bitmap), ("grouped", grouped), ("grouped-32", hs.bitmap_to_grouped(bitmap))):
                got = gpu_spmm(torch_cuda, hs, fmt, B, N)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "%s %dx%d N=%d" % (name, rows, cols, N)
        # Sparse windows: the bitmap arrays go to the device as they are (no expansion on the
        # host); the kernels that read plain tiles (N = 8: the all-shapes kernel) run on what a kernel expanded
        # there, and with the bitmap stream forced the gather kernels read the caller's own words and elements.
        sparse = plain["total_tiles"] < 1.2 * plain["eff_row_windows"] * ((cols + 127) // 128)     # (else: LDS-staging stream, built on the host)
        plan = hs.Plan(bitmap)
        assert plan.info()["bitmap_from_caller"] == (1 if sparse else 0), (rows, cols)
        plan.close()
        if sparse:
            os.environ["HSPMM_GATHER_BITMAP"] = "1"
            try:
                forced = hs.Plan(bitmap)
            finally:
                os.environ.pop("HSPMM_GATHER_BITMAP", None)
            info = forced.info()
            assert info["bitmap_from_caller"] == 1 and info["gather_bitmap"] == 1
            for N in (64, 128):
                B = make_b(rng, cols, N, dtype)
                got = gpu_spmm(torch_cuda, hs, bitmap, B, N, plan=forced)
                assert forced.info()["last_kernel_family"] == 2
                assert np.array_equal(got.view(np.uint8), gpu_spmm(torch_cuda, hs, plain, B, N).view(np.uint8))
            forced.close()
            # a tile whose bits and nnzOffset span disagree is refused on this path as on the other
            broken = dict(bitmap)
            broken["tcBit"] = bitmap["tcBit"].copy()
            broken["tcBit"][0] ^= np.uint64(1) << np.uint64(63)
            with pytest.raises(hs.HspmmError):
                hs.Plan(broken)
    # golden file through the compressed format
    A = hs.mtx_load(os.path.join(GOLD, "tiny.mtx"), dtype)
    A["dtype"] = dtype
    bitmap = hs.csr_to_bitmap(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], dtype)
    B = make_b(rng, A["cols"], 32, dtype)
    ref, mag = oracle_spmm(oracle, A, B, 32)
    assert_parity(gpu_spmm(torch_cuda, hs, bitmap, B, 32), ref, mag, dtype, "tiny.mtx bitmap")


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_plans_from_transposed_tiles_and_from_tiles_four_columns_wide(torch_cuda, hs, oracle, dtype):
    """The tile layouts of the reference's two optional build switches describe the same matrix:
    tiles written column by column (-DSPARSE_A_TRANSPOSE, src/utils/convert.h:207-209), by the
    library's converter and by the oracle's, and for fp32 storage the 8 x 4 tiles of -DMMA_M16N8K4
    (src/common.h:28-35), by both converters as well.  Their plans give bit for bit what the plan of the
    default layout gives, and that agrees with the oracle."""
    rng = np.random.default_rng(190 + dtype)
    for rows, cols, dens, erp, heavy in [(27, 100, 0.1, 0.5, ()), (300, 3000, 0.004, 0.2, (5, 100, 101, 299)),
                                         (1000, 700, 0.01, 0.6, (512,)), (64, 64, 1.0, 0.0, ())]:
        A = random_csr(rng, rows, cols, dens, dtype, erp, heavy)
        plain = convert(hs, A)
        csr = (rows, cols, A["row_ptr"], A["col_idx"], A["values"])
        layouts = [("transposed", hs.csr_to_btcf(*csr, dtype, transpose=True))]
        assert layouts[0][1]["transposed"] and not np.array_equal(layouts[0][1]["data"], plain["data"])
        if dtype == 1:
            layouts += [("library 8x4", hs.csr_to_btcf(*csr, dtype, cw=4)),
                        ("library 8x4 transposed", hs.csr_to_btcf(*csr, dtype, transpose=True, cw=4))]
            assert layouts[1][1]["cw"] == 4 and layouts[1][1]["total_tiles"] >= plain["total_tiles"]
        for name, kw in (("oracle transposed", dict(transpose=True)), ("8x4", dict(cw=4)),
                         ("8x4 transposed", dict(cw=4, transpose=True))):
            if "cw" in kw and dtype != 1:
                continue
            o = dict(oracle.csr_to_btcf(*csr, DT[dtype], **kw))
            o.update(dtype=dtype, transposed=bool(kw.get("transpose")))
            if "cw" in kw:
                assert o["cw"] == 4 and o["total_tiles"] >= plain["total_tiles"]
            layouts.append((name, o))
        for N in (8, 64, 136):
            B = make_b(rng, cols, N, dtype)
            want = gpu_spmm(torch_cuda, hs, plain, B, N)
            ref, mag = oracle_spmm(oracle, A, B, N)
            assert_parity(want, ref, mag, dtype, "plain %dx%d N=%d" % (rows, cols, N))
            for name, fmt in layouts:
                got = gpu_spmm(torch_cuda, hs, fmt, B, N)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "%s %dx%d N=%d" % (name, rows, cols, N)
    # what the entry point refuses
    bad = dict(plain, cw=4)
    if dtype != 1:
        with pytest.raises(hs.HspmmError):
            hs.Plan(bad)


def test_partition_exported_as_groups_round_trips(torch_cuda, hs, oracle):
    """hspmm_partition_as_groups writes the plan's balanced partition in the reference's grouped form
    (GBTCF_MTX, src/utils/class.h:93-108): every group is the piece of one window that one wave walks, windows
    cut across waves are marked atomic, and the groups together with the tile arrays are a matrix that
    hspmm_create_grouped takes back - same product, bit for bit."""
    rng = np.random.default_rng(77)
    A = random_csr(rng, 300, 3000, 0.004, 0, 0.2, (5, 100, 101, 299))
    plain = convert(hs, A)
    bitmap = hs.csr_to_bitmap(300, 3000, A["row_ptr"], A["col_idx"], A["values"], 0)
    hs.configure(producer_warp_group_num=16)            # many short ranges: the heavy windows are cut
    try:
        plan = hs.Plan(plain)
    finally:
        hs.configure()
    assert plan.info()["n_split_windows"] > 0
    g = plan.partition_as_groups()
    ranges = plan.partition()
    go, T = g["groupOffset"].astype(np.int64), plain["total_tiles"]
    assert go[0] == 0 and go[-1] == T and (np.diff(go) > 0).all()
    assert set(plain["rowOffset"].tolist()) <= set(go.tolist())                     # no group straddles a window
    assert set(ranges[:, 0].tolist()) <= set(go.tolist())                           # nor a range
    window_of_group = np.searchsorted(plain["rowOffset"], go[:-1], side="right") - 1
    assert np.array_equal(g["rowIdx"], plain["rowIdx"][window_of_group])
    groups_per_window = np.bincount(window_of_group, minlength=plain["eff_row_windows"])
    assert np.array_equal(g["atomic"].astype(bool), groups_per_window[window_of_group] > 1)
    assert g["atomic"].sum() >= 2 * plan.info()["n_split_windows"]
    plan.close()
    grouped = {k: bitmap[k] for k in ("rows", "cols", "nnzs", "dtype", "cw", "nnzOffset", "tcA2B", "tcBit", "data")}
    grouped.update(g, tgl=0, total_row_windows=g["total_groups"] + 1, eff_row_windows=g["total_groups"] + 1)
    for N in (8, 64):
        B = make_b(rng, 3000, N, 0)
        want = gpu_spmm(torch_cuda, hs, plain, B, N)
        assert np.array_equal(gpu_spmm(torch_cuda, hs, grouped, B, N), want)
    # A plan that walks pairs of windows (equal column lists merged) exports the balanced partition of the caller's
    # single windows: groups of the caller's tiles again, which hspmm_create_grouped takes back.
    P = _block_matrix(rng, 256, 1200, 16, 16, 0.5, 0)                                   # block-clustered: windows pair up
    pplain = convert(hs, P)
    pbitmap = hs.csr_to_bitmap(256, 1200, P["row_ptr"], P["col_idx"], P["values"], 0)
    hs.configure(producer_warp_group_num=16)
    try:
        pairs = hs.Plan(pplain)
    finally:
        hs.configure()
    assert pairs.info()["n_paired_units"] > 0
    g = pairs.partition_as_groups()
    pairs.close()
    go = g["groupOffset"].astype(np.int64)
    assert go[0] == 0 and go[-1] == pplain["total_tiles"] and (np.diff(go) > 0).all()
    assert set(pplain["rowOffset"].tolist()) <= set(go.tolist())
    window_of_group = np.searchsorted(pplain["rowOffset"], go[:-1], side="right") - 1
    assert np.array_equal(g["rowIdx"], pplain["rowIdx"][window_of_group])
    groups_per_window = np.bincount(window_of_group, minlength=pplain["eff_row_windows"])
    assert np.array_equal(g["atomic"].astype(bool), groups_per_window[window_of_group] > 1)
    pgrouped = {k: pbitmap[k] for k in ("rows", "cols", "nnzs", "dtype", "cw", "nnzOffset", "tcA2B", "tcBit", "data")}
    pgrouped.update(g, tgl=0, total_row_windows=g["total_groups"] + 1, eff_row_windows=g["total_groups"] + 1)
    B = make_b(rng, 1200, 64, 0)
    ref, mag = oracle_spmm(oracle, P, B, 64)
    assert_parity(gpu_spmm(torch_cuda, hs, pgrouped, B, 64), ref, mag, 0, "groups of a plan that pairs windows")


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_plans_that_cut_windows_only_where_the_callers_groups_end(torch_cuda, hs, oracle, dtype):
    """hspmm_set_group_cuts(1): the waves of the gather kernels walk whole groups of the caller's grouped matrix
    (GBTCF_MTX, reference src/utils/convert.h:245-259) - a heavy window is cut at group ends only, its partial sums
    are added in group order.  Agrees with the oracle; bit for bit with the plain plan on inputs whose sums are exact."""
    rng = np.random.default_rng(400 + dtype)
    rows, cols = 300, 6000
    A = random_csr(rng, rows, cols, 0.002, dtype, 0.2, (5, 100, 101, 299))
    bitmap = hs.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype)
    grouped = hs.bitmap_to_grouped(bitmap, min_len=7)
    assert grouped["atomic"].any()
    hs.configure(producer_warp_group_num=16)            # many short ranges: the heavy windows are cut
    hs.set_group_cuts(1)
    if dtype == 1:
        hs.set_kernel_mode(3)                           # (fp32 storage: by default the LDS-staging kernels, which walk no groups)
    try:
        kept = hs.Plan(grouped)
        hs.set_group_cuts(0)
        free = hs.Plan(grouped)
        _run_group_cut_checks(torch_cuda, hs, oracle, rng, A, grouped, kept, free, dtype)
    finally:
        hs.set_group_cuts(0)
        hs.set_kernel_mode(0)
        hs.configure()


def _run_group_cut_checks(torch_cuda, hs, oracle, rng, A, grouped, kept, free, dtype):
    rows, cols = A["rows"], A["cols"]
    assert kept.info()["group_cuts_kept"] == 1 and free.info()["group_cuts_kept"] == 0
    assert kept.info()["n_split_windows"] > 0
    go = grouped["groupOffset"]
    assert np.isin(kept.partition()[:, 0], go).all()
    assert not np.isin(free.partition()[:, 0], go).all()                          # the cost model cuts elsewhere
    assert np.isin(kept.partition_as_groups()["groupOffset"], go).all()            # what it walks are runs of whole groups
    for N in (64, 128, 8):
        B = make_b(rng, cols, N, dtype)
        ref, mag = oracle_spmm(oracle, A, B, N)
        got = gpu_spmm(torch_cuda, hs, grouped, B, N, plan=kept)
        assert_parity(got, ref, mag, dtype, "group cuts N=%d" % N)
        assert N == 8 or kept.info()["last_kernel_family"] == 2
    # small integers: every product and sum is exact, so the order of the additions cannot show
    E = dict(A)
    E["values"] = encode(rng.integers(-3, 4, A["nnzs"]).astype(np.float32), dtype)
    eb = hs.csr_to_bitmap(rows, cols, E["row_ptr"], E["col_idx"], E["values"], dtype)
    eg = hs.bitmap_to_grouped(eb, min_len=7)
    B = encode(rng.integers(-4, 5, (cols, 64)).astype(np.float32), dtype)
    hs.set_group_cuts(1)
    kept_exact = hs.Plan(eg)
    hs.set_group_cuts(0)
    assert kept_exact.info()["group_cuts_kept"] == 1
    got = gpu_spmm(torch_cuda, hs, eg, B, 64, plan=kept_exact)
    want = gpu_spmm(torch_cuda, hs, convert(hs, E), B, 64)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    for plan in (kept, free, kept_exact):
        plan.close()
    # windows merged through equal column lists are not the caller's tiles any more: the cuts are dropped
    P = random_csr(rng, 64, 64, 1.0, dtype)
    pg = hs.bitmap_to_grouped(hs.csr_to_bitmap(64, 64, P["row_ptr"], P["col_idx"], P["values"], dtype), min_len=1)
    hs.set_group_cuts(1)
    try:
        merged = hs.Plan(pg)
    finally:
        hs.set_group_cuts(0)
    if merged.info()["n_paired_units"]:
        assert merged.info()["group_cuts_kept"] == 0
    merged.close()


PANEL_SHAPES = [
    # rows, cols, density, empty-row probability, heavy rows
    (8, 16, 1.0, 0.0, ()),                      # one window, one panel
    (27, 100, 0.3, 0.3, ()),                    # ragged last window, one panel
    (130, 257, 0.2, 0.3, ()),                   # three panels, the last one a single column
    (300, 1000, 0.1, 0.2, (5, 100, 299)),
    (1000, 700, 0.01, 0.6, (512,)),             # most units have no step in most panels
]


@pytest.mark.parametrize("dtype", [0, 1, 2])
@pytest.mark.parametrize("shape", PANEL_SHAPES)
def test_lds_panel_kernels_on_every_shape(torch_cuda, hs, oracle, dtype, shape):
    rows, cols, dens, erp, heavy = shape
    rng = np.random.default_rng(hash((rows, cols, dtype, 4)) & 0xFFFF)
    A = random_csr(rng, rows, cols, dens, dtype, erp, heavy)
    b = convert(hs, A)
    block = 64 if dtype == 1 else 128
    # units: consumer waves of a workgroup that get a unit (HSPMM_PANEL_UNITS_PER_GROUP; the kernels have 8, 12 or 14)
    cases = [(4, u, c) for u, c in (("", ""), ("12", ""), ("5", ""), ("7", "2"), ("1", "1"), ("14", "3"), ("3", "1000"))]
    if dtype == 1:                              # fp32 products: the 4x4x1 / 16x16x4 MFMA forms
        cases += [(5, "", ""), (5, "12", "2"), (5, "6", "3"), (5, "14", "1")]
    for mode, units, chunks in cases:
        if units:
            os.environ["HSPMM_PANEL_UNITS_PER_GROUP"] = units
        if chunks:
            os.environ["HSPMM_PANEL_CHUNKS"] = chunks
        hs.set_kernel_mode(mode)
        try:
            plan = hs.Plan(b)
            info = plan.info()
            # a step is 32 columns (4 fp32 tiles, 2 16-bit tiles) or, with fp32 products, one tile
            per_step = 1 if mode == 5 else 4 if dtype == 1 else 2
            panel_rows = 128 if mode == 5 else 256      # the fp32 MFMA forms keep panels of 128 columns
            assert info["n_panels"] == (cols + panel_rows - 1) // panel_rows
            # (adjacent windows with much the same columns may have been given one list: up to four windows per step)
            assert info["n_panel_steps"] >= info["total_tiles"] // (4 * per_step)
            # (any N of one block at least: the last block moves back to end with the row; fp32 storage in bf16 parts
            # also takes one partly empty block from 16 features on when its rows are whole 16-byte pieces)
            ragged = (block + 16, 3 * block - 16, block + 1, 2 * block + 7, 5 * block - 1)
            if dtype == 1 and mode != 5:
                ragged += (16, 48, 20)
            if dtype != 1:
                ragged += (block + 8, 3 * block - 24, 2 * block + 2)
            for N in (block, 2 * block, 5 * block) + ragged:
                B = make_b(rng, cols, N, dtype)
                got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
                ref, mag = oracle_spmm(oracle, A, B, N)
                assert_parity(got, ref, mag, dtype, "panel mode %d units %s chunks %s shape %s N=%d" % (mode, units, chunks, shape[:2], N))
                assert plan.info()["last_kernel_family"] == 3          # the LDS-staging kernels did run
            # a feature dimension the panel kernels do not take falls back to the gather kernels
            B = make_b(rng, cols, 22, dtype)
            got = gpu_spmm(torch_cuda, hs, b, B, 22, plan=plan)
            ref, mag = oracle_spmm(oracle, A, B, 22)
            assert_parity(got, ref, mag, dtype, "panel plan, N=22", tight=got.size >= 10000)   # (a share of 99.9 % needs that many)
            assert plan.info()["last_kernel_family"] == 2
            plan.close()
        finally:
            hs.set_kernel_mode(0)
            os.environ.pop("HSPMM_PANEL_UNITS_PER_GROUP", None)
            os.environ.pop("HSPMM_PANEL_CHUNKS", None)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_lds_panel_kernels_exact_and_paired(torch_cuda, hs, oracle, dtype):
    """Block-clustered matrices (paired windows) and exact integer arithmetic: the panel
    kernels must give the one rounding of the exact result, like the gather kernels."""
    rng = np.random.default_rng(70 + dtype)
    block = 64 if dtype == 1 else 128
    A = _block_matrix(rng, 203, 900, 16, 16, 0.5, dtype)
    b = convert(hs, A)
    D = rng.integers(-3, 4, (120, 700)) * (rng.random((120, 700)) < 0.3)
    rp = np.zeros(121, np.uint32)
    ci, vv = [], []
    for r in range(120):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    E = dict(rows=120, cols=700, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32),
             values=encode(np.array(vv, np.float32), dtype))
    e = convert(hs, E)
    try:
        for mode in ((4, 5) if dtype == 1 else (4,)):
            hs.set_kernel_mode(mode)
            for pairing in (0, 1, 2):
                hs.set_window_pairing(pairing)
                plan = hs.Plan(b)
                assert plan.info()["n_panels"] == (8 if mode == 5 else 4)
                if pairing != 1:
                    assert plan.info()["n_paired_units"] > 0
                for N in (block, 3 * block):
                    B = make_b(rng, 900, N, dtype)
                    got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
                    ref, mag = oracle_spmm(oracle, A, B, N)
                    assert_parity(got, ref, mag, dtype, "paired panel mode %d pairing %d N=%d" % (mode, pairing, N))
                plan.close()
            hs.set_window_pairing(0)
            plan = hs.Plan(e)
            Bm = rng.integers(-4, 5, (700, 2 * block))
            got = gpu_spmm(torch_cuda, hs, e, encode(Bm, dtype), 2 * block, plan=plan)
            assert np.array_equal(got, encode(D @ Bm, dtype))
            plan.close()
    finally:
        hs.set_kernel_mode(0)
        hs.set_window_pairing(0)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_long_units_are_walked_by_one_workgroup_each(torch_cuda, hs, oracle, dtype):
    """Matrices whose units are all long (block-clustered weights at a small feature dimension): every
    unit is cut into the ranges of one workgroup, which adds the partial sums itself and stores the
    unit - one kernel, although the balanced partition of the same plan cuts every unit.  Exact
    integers: the result must be the one rounding of the exact product, as from every other path."""
    torch = torch_cuda
    rng = np.random.default_rng(90 + dtype)
    rows, cols = 75, 8192                                   # 10 windows (the last with 3 rows), 256-tile units
    keep = rng.random((5, cols // 16)) < 0.5                # 16-row blocks: pairs of windows with one column list
    D = np.zeros((rows, cols), np.int64)
    for r in range(rows):
        cols_kept = np.repeat(keep[r // 16], 16)
        D[r, cols_kept] = rng.integers(-3, 4, int(cols_kept.sum()))
    D[32:40] = 0                                            # an empty window: the pair around it is broken
    rp = np.zeros(rows + 1, np.uint32)
    ci, vv = [], []
    for r in range(rows):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    A = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32),
             values=encode(np.array(vv, np.float32), dtype))
    b = convert(hs, A)
    for pairing in (0, 1):
        hs.set_window_pairing(pairing)
        if dtype == 1:
            hs.set_kernel_mode(3)                           # (fp32 storage: the LDS-staging kernels would take N = 16 and 48)
        try:
            plan = hs.Plan(b)
        finally:
            hs.set_window_pairing(0)
            hs.set_kernel_mode(0)
        assert plan.info()["n_split_windows"] > 0           # the balanced partition cuts units
        for N in (8, 16, 48, 56 if dtype == 1 else 64):
            Bm = rng.integers(-4, 5, (cols, N))
            got = gpu_spmm(torch, hs, b, encode(Bm, dtype), N, plan=plan)
            assert np.array_equal(got, encode(D @ Bm, dtype)), (pairing, N)
            assert plan.info()["last_kernel_family"] == 2
            tt = torch.float32 if dtype == 1 else torch.int16
            dB = torch.zeros((cols, N), dtype=tt, device="cuda")
            dC = torch.empty((rows, N), dtype=tt, device="cuda")
            main_ms, sum_ms = plan.profile(dB.data_ptr(), dC.data_ptr(), N, runs=2)
            assert main_ms > 0 and sum_ms == 0, "a second kernel ran"
        plan.close()


@pytest.mark.parametrize("dtype", [0, 1])
def test_partial_sums_added_inside_the_main_kernel(torch_cuda, hs, oracle, dtype):
    """The wave that brings the last partial sum of a cut unit, or of a unit's chunks of panels, adds them
    in the fixed order and stores the unit (the default of the LDS-staging kernels, and of the gather kernels
    where few units are cut; HSPMM_FUSED_FIXUP = 1 / 0 forces it / the second launch): the same bits launch
    after launch, whoever arrives last, and for chunks of panels the bits of the two-launch path."""
    torch = torch_cuda
    rng = np.random.default_rng(33 + dtype)
    block = 64 if dtype == 1 else 128
    sparse = random_csr(rng, 300, 3000, 0.004, dtype, 0.2, (5, 100, 101, 299))     # heavy windows: cut units
    dense = random_csr(rng, 300, 3000, 0.1, dtype, 0.1)                             # LDS-staging kernels
    # (fp32 storage: every N of whole 16-byte pieces per row goes to the LDS-staging kernels when the plan has them)
    for A, N, family in ((sparse, 42 if dtype == 1 else 64, 2), (dense, block, 3)):
        b = convert(hs, A)
        B = make_b(rng, 3000, N, dtype)
        hs.configure(producer_warp_group_num=16)
        os.environ["HSPMM_PANEL_CHUNKS"] = "3"
        try:
            os.environ["HSPMM_FUSED_FIXUP"] = "0"
            try:
                two = hs.Plan(b)
            finally:
                os.environ.pop("HSPMM_FUSED_FIXUP", None)
            want = gpu_spmm(torch, hs, b, B, N, plan=two)
            tt = torch.float32 if dtype == 1 else torch.int16
            dB = torch.zeros((3000, N), dtype=tt, device="cuda")
            dC = torch.empty((300, N), dtype=tt, device="cuda")
            main_ms, sum_ms = two.profile(dB.data_ptr(), dC.data_ptr(), N, runs=2)
            assert main_ms > 0 and sum_ms > 0                  # two launches
            two.close()
            os.environ["HSPMM_FUSED_FIXUP"] = "1"
            try:
                plan = hs.Plan(b)
            finally:
                os.environ.pop("HSPMM_FUSED_FIXUP", None)
            ref, mag = oracle_spmm(oracle, A, B, N)
            first = gpu_spmm(torch, hs, b, B, N, plan=plan)
            assert_parity(first, ref, mag, dtype, "sums added in the main kernel")
            if family == 3:             # the chunk order is the same in both paths; the gather kernels' two-kernel
                assert np.array_equal(first, want)      # path adds four ranges per workgroup first
            for _ in range(3):
                assert np.array_equal(gpu_spmm(torch, hs, b, B, N, plan=plan), first)
            assert plan.info()["last_kernel_family"] == family
            tt = torch.float32 if dtype == 1 else torch.int16
            dB = torch.zeros((3000, N), dtype=tt, device="cuda")
            dC = torch.empty((300, N), dtype=tt, device="cuda")
            main_ms, sum_ms = plan.profile(dB.data_ptr(), dC.data_ptr(), N, runs=2)
            assert main_ms > 0 and sum_ms == 0
            plan.close()
        finally:
            hs.configure()
            os.environ.pop("HSPMM_PANEL_CHUNKS", None)
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(want, ref, mag, dtype, "two-kernel path")


def test_error_of_the_three_product_fp32_arithmetic_against_fp64(torch_cuda, hs):
    """The LDS-staging kernels multiply fp32 storage as bf16 parts in three products (a_lo b_lo left out):
    against an fp64 product the error stays below 2^-16 sum |a||b| on normal entries and below the hard bound
    2^-14 sum |a||b| on the adversarial input - every factor positive with all low mantissa bits set, so that
    nothing cancels and every left-out product is as large as it can be; with fp32 products (kernel mode 5)
    it is rounding of the fp32 sums only."""
    rng = np.random.default_rng(404)
    rows, cols, N = 512, 2048, 64
    mask = rng.random((rows, cols)) < 0.1
    rp = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.uint32)
    ci = np.nonzero(mask)[1].astype(np.uint32)
    all_ones = np.float32(np.frombuffer(np.uint32(0x3FFFFFFF).tobytes(), np.float32)[0])      # 1.9999999
    cases = {
        "normal": (rng.normal(size=ci.size).astype(np.float32), rng.normal(size=(cols, N)).astype(np.float32), 2.0 ** -16),
        "adversarial": ((all_ones * np.exp2(rng.integers(-3, 4, ci.size))).astype(np.float32),
                        (all_ones * np.exp2(rng.integers(-3, 4, (cols, N)))).astype(np.float32), 2.0 ** -14),
    }
    for name, (vals, B, bound) in cases.items():
        D = np.zeros((rows, cols), np.float64)
        D[mask] = vals
        ref = D @ B.astype(np.float64)
        mag = np.abs(D) @ np.abs(B).astype(np.float64)
        A = dict(rows=rows, cols=cols, row_ptr=rp, col_idx=ci, values=vals, dtype=1)
        b = convert(hs, A)
        for mode, limit in ((0, bound), (5, 2.0 ** -20)):
            hs.set_kernel_mode(mode)
            try:
                plan = hs.Plan(b)
                got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
                assert plan.info()["last_kernel_family"] == 3, (name, mode)
                plan.close()
            finally:
                hs.set_kernel_mode(0)
            worst = float((np.abs(got.astype(np.float64) - ref) / mag).max())
            assert worst <= limit, "%s, kernel mode %d: %.3g sum |a||b| (2^%.1f)" % (name, mode, worst, np.log2(worst))
            if mode == 0 and name == "adversarial":
                assert worst > 2.0 ** -17        # the left-out product is there: this input does exercise the bound


def test_lds_panel_kernels_are_chosen_for_dense_windows_only(torch_cuda, hs):
    from hopper_spmm_amd import generators as G
    dense = G.make_config(4, 8)["A"]            # block-clustered: every window meets half of all columns
    sparse = G.make_config(1, 8)["A"]           # ~16 entries per row
    assert hs.Plan(convert(hs, dense)).info()["n_panels"] > 0
    assert hs.Plan(convert(hs, sparse)).info()["n_panels"] == 0


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_adjacent_windows_with_overlapping_columns_share_units(torch_cuda, hs, oracle, dtype):
    """In the LDS-panel kernels' copy of the matrix adjacent windows are given the union of their
    column lists and run as one unit - pairs, and with pairing mode 2 (or on matrices large enough
    to fill the GPU that way) groups of three and four windows: same product (the added entries are
    zeros), also when the panels are cut into chunks whose sums a second kernel adds; the other
    kernel families keep the caller's windows."""
    rng = np.random.default_rng(40 + dtype)
    rows, cols = 203, 1500
    D = rng.integers(-3, 4, (rows, cols)) * (rng.random((rows, cols)) < 0.25)
    D[64:80] = 0                                        # two empty windows in the middle
    D[136:144] = 0                                      # and one that leaves seven windows in a row: 4 + 3
    D[100, :] = rng.integers(1, 3, cols)                # a full row
    rp = np.zeros(rows + 1, np.uint32)
    ci, vv = [], []
    for r in range(rows):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    A = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32),
             values=encode(np.array(vv, np.float32), dtype))
    b = convert(hs, A)
    block = 64 if dtype == 1 else 128
    for mode in (0, 1, 2, 3, 4, 5):
        for pairing in (0, 1, 2):
            hs.set_kernel_mode(mode)
            hs.set_window_pairing(pairing)
            try:
                plan = hs.Plan(b)
            finally:
                hs.set_kernel_mode(0)
                hs.set_window_pairing(0)
            info = plan.info()
            assert info["total_tiles"] == b["total_tiles"] and info["n_paired_units"] == 0
            grouped = mode in (0, 4) or (mode == 5 and dtype != 1)     # a panel stream built on the 16-bit MFMA
            if grouped:
                assert info["n_panels"] > 0
                assert (info["n_panel_paired_units"] > 0) == (pairing != 1), (mode, pairing, info)
                # (fp32 storage in bf16 parts has units of three and four windows in builds with EXPERIMENTAL=1 only)
                wide = pairing == 2 and (dtype != 1 or hs.has_experimental())
                assert (info["n_panel_wide_units"] > 0) == wide, (mode, pairing, info)
                if wide:                # 8, 7 and 8 windows between the gaps: two fours, a four and a three, two fours
                    assert info["n_panel_units"] == 6 and info["n_panel_wide_units"] == 6, info
            for chunks in (None, "2") if grouped else (None,):
                if chunks:
                    os.environ["HSPMM_PANEL_CHUNKS"] = chunks
                try:
                    for N in (block, 2 * block, 24):
                        Bm = rng.integers(-4, 5, (cols, N))
                        got = gpu_spmm(torch_cuda, hs, b, encode(Bm, dtype), N, plan=plan)
                        assert np.array_equal(got, encode(D @ Bm, dtype)), (mode, pairing, chunks, N)
                finally:
                    os.environ.pop("HSPMM_PANEL_CHUNKS", None)
            plan.close()


@pytest.mark.parametrize("dtype", [0, 2])
def test_units_of_four_windows_are_chosen_for_large_pruned_matrices(torch_cuda, hs, oracle, dtype):
    """A 16-bit matrix with dense windows and enough rows to fill the GPU with units of 32 rows gets
    them without being asked; a smaller one, and fp32 storage, keep pairs."""
    from hopper_spmm_amd import generators as G
    rows, cols, N = 13312, 1024, 256                     # 416 units of four windows >= 1.5 x 256 compute units
    A = G.pruned_weight(rows, cols, 0.10, 77, dtype=dtype)
    b = convert(hs, A)
    plan = hs.Plan(b)
    info = plan.info()
    assert info["n_panels"] == 4 and info["n_panel_units"] == rows // 32 == info["n_panel_wide_units"], info
    rng = np.random.default_rng(5)
    B = make_b(rng, cols, N, dtype)
    got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
    plan.close()
    ref, mag = oracle_spmm(oracle, A, B, N)
    assert_parity(got, ref, mag, dtype, "units of four windows")
    small = G.pruned_weight(4096, cols, 0.10, 78, dtype=dtype)
    assert hs.Plan(convert(hs, small)).info()["n_panel_wide_units"] == 0
    f32 = G.pruned_weight(rows, cols, 0.10, 77, dtype=1)
    info = hs.Plan(convert(hs, f32)).info()
    assert info["n_panels"] > 0 and info["n_panel_paired_units"] > 0 and info["n_panel_wide_units"] == 0


@pytest.mark.parametrize("seed,large", [(11, False), (12, False), (13, False), (14, True)])
def test_seeded_sweep_of_shapes_formats_and_kernel_choices(torch_cuda, hs, oracle, seed, large):
    """Seeded combinations (150 per seed; 80 for the sweep over larger shapes, whose matrices span
    many column panels and several workgroups) of element type, shape, density, empty and heavy rows,
    kernel mode, window pairing, input format (plain / bitmap / grouped), prefetch depth,
    partition granularity and feature dimension, each compared with the oracle."""
    rng = np.random.default_rng(seed)
    for case in range(80 if large else 150):
        dtype = int(rng.integers(0, 3))
        if large:
            rows = int(rng.choice([513, 1000, 2049, 4100]))
            cols = int(rng.choice([255, 1025, 4097, 9000, 20001]))
            dens = float(rng.choice([0.001, 0.01, 0.05, 0.2]))
        else:
            rows = int(rng.choice([1, 7, 8, 9, 31, 64, 129, 300, 777]))
            cols = int(rng.choice([1, 5, 16, 17, 127, 128, 129, 500, 2049, 6000]))
            dens = float(rng.choice([0.002, 0.02, 0.1, 0.4, 0.9]))
        erp = float(rng.choice([0.0, 0.3, 0.8]))
        heavy = tuple(int(x) for x in rng.integers(0, rows, int(rng.integers(0, 3)))) if rows > 8 else ()
        A = random_csr(rng, rows, cols, dens, dtype, erp, heavy)
        mode = int(rng.choice([0, 0, 2, 3, 4, 4, 5]))
        pairing = int(rng.integers(0, 3))
        fmt = int(rng.integers(0, 3))
        stages = built_depth(hs, int(rng.choice([0, 0, 1, 2, 4])))
        ranges_per_simd = int(rng.choice([0, 0, 1, 16]))
        if mode >= 4 and large:
            N = int(rng.choice([64, 128, 320, 512])) if dtype == 1 else int(rng.choice([128, 256, 640, 1024]))
        elif mode >= 4:
            N = int(rng.choice([64, 128, 192, 256, 384])) if dtype == 1 else int(rng.choice([128, 256, 384]))
        else:
            N = int(rng.choice([1, 2, 3, 8, 16, 24, 32, 40, 64, 96, 128, 136, 256, 320]))
        what = "seed %d case %d: type %s %dx%d density %g empty %g heavy %s mode %d pairing %d format %d stages %d rps %d N %d" % (
            seed, case, DT[dtype], rows, cols, dens, erp, heavy, mode, pairing, fmt, stages, ranges_per_simd, N)
        hs.set_kernel_mode(mode)
        hs.set_window_pairing(pairing)
        hs.configure(buffer_stage=stages, producer_warp_group_num=ranges_per_simd)
        try:
            if fmt == 0:
                b = convert(hs, A)
            else:
                b = hs.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype)
                if fmt == 2:
                    b = hs.bitmap_to_grouped(b, int(rng.choice([1, 4, 32])))
            plan = hs.Plan(b)
        finally:
            hs.set_kernel_mode(0)
            hs.set_window_pairing(0)
            hs.configure()
        B = make_b(rng, cols, N, dtype)
        got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
        plan.close()
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(got, ref, mag, dtype, what, tight=False)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_seeded_sweep_of_stream_modes_group_cuts_and_tuning_overrides(torch_cuda, hs, oracle, seed):
    """As the sweep above (120 combinations per seed), with the choices it leaves at their defaults drawn as well:
    the stream mode of the LDS-staging kernels, grouped input that keeps the caller's cuts, tiles written column
    by column, and the overrides read from the environment at plan creation (bitmap stream of the gather kernels,
    feature blocks dealt out by XCD, partial sums added inside the main kernel, one workgroup per unit for small
    matrices, windows per unit of the panel stream), feature dimensions that end inside a block of features or
    are odd, and B and C that start anywhere on an element (nothing around C may be written)."""
    knobs = ("HSPMM_GATHER_BITMAP", "HSPMM_XCD_SPLIT", "HSPMM_FUSED_FIXUP", "HSPMM_ALIGNED_SMALL", "HSPMM_PANEL_MAX_WINDOWS")
    rng = np.random.default_rng(seed)
    for case in range(120):
        dtype = int(rng.integers(0, 3))
        rows = int(rng.choice([1, 7, 8, 9, 15, 16, 17, 31, 64, 129, 300, 777]))
        cols = int(rng.choice([1, 5, 16, 17, 31, 33, 127, 128, 129, 255, 257, 500, 2049, 6000]))
        dens = float(rng.choice([0.002, 0.02, 0.1, 0.4, 0.9, 1.0]))
        erp = float(rng.choice([0.0, 0.3, 0.8]))
        heavy = tuple(int(x) for x in rng.integers(0, rows, int(rng.integers(0, 3)))) if rows > 8 else ()
        A = random_csr(rng, rows, cols, dens, dtype, erp, heavy)
        mode = int(rng.choice([0, 0, 0, 2, 3, 4, 4, 5]))
        pairing = int(rng.integers(0, 3))
        fmt = int(rng.integers(0, 5))          # plain, bitmap, grouped, grouped with its cuts kept, column by column
        stages = built_depth(hs, int(rng.choice([0, 0, 0, 1, 2, 4])))
        ranges_per_simd = int(rng.choice([0, 0, 1, 16]))
        stream = int(rng.choice([0, 0, 1, 2]))
        if not hs.has_experimental():
            stream = 0                         # (stream modes 1 and 2 are built with EXPERIMENTAL=1 only)
        env = {}
        for name, chance, values in zip(knobs, (0.3, 0.3, 0.3, 0.2, 0.2), ([0, 1], [0, 1], [0, 1], [0, 4, 8], [2, 4])):
            if rng.random() < chance:
                env[name] = str(int(rng.choice(values)))
        if mode >= 4 and dtype == 1:
            N = int(rng.choice([16, 20, 48, 64, 65, 67, 68, 80, 100, 127, 128, 130, 144, 192, 250, 256, 320, 512]))
        elif mode >= 4:
            N = int(rng.choice([128, 129, 130, 136, 144, 200, 208, 250, 255, 256, 384, 400, 640, 1000, 1001, 1024]))
        else:
            N = int(rng.choice([1, 2, 3, 6, 7, 8, 10, 16, 24, 30, 32, 40, 64, 96, 100, 127, 128, 130, 136, 250, 256, 320, 512, 1000, 1002]))
        element = 4 if dtype == 1 else 2
        offsets = tuple(int(rng.choice([0, 0, 1, 2, 3, 4, 5, 8])) * element if rng.random() < 0.5 else 0 for _ in range(2))
        what = "seed %d case %d: type %s %dx%d density %g empty %g heavy %s mode %d pairing %d format %d stages %d rps %d stream %d %s N %d B, C %s bytes in" % (
            seed, case, DT[dtype], rows, cols, dens, erp, heavy, mode, pairing, fmt, stages, ranges_per_simd, stream, env, N, offsets)
        hs.set_kernel_mode(mode)
        hs.set_window_pairing(pairing)
        hs.set_panel_stream(stream)
        hs.configure(buffer_stage=stages, producer_warp_group_num=ranges_per_simd)
        os.environ.update(env)
        try:
            if fmt == 0:
                b = convert(hs, A)
            elif fmt == 4:
                b = hs.csr_to_btcf(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype, transpose=True)
            else:
                b = hs.csr_to_bitmap(rows, cols, A["row_ptr"], A["col_idx"], A["values"], dtype)
                if fmt >= 2:
                    b = hs.bitmap_to_grouped(b, int(rng.choice([1, 4, 32])))
                    hs.set_group_cuts(1 if fmt == 3 else 0)
            plan = hs.Plan(b)
        finally:
            hs.set_kernel_mode(0)
            hs.set_window_pairing(0)
            hs.set_panel_stream(0)
            hs.set_group_cuts(0)
            hs.configure()
            for name in knobs:
                os.environ.pop(name, None)
        B = make_b(rng, cols, N, dtype)
        got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan, offsets=offsets)
        plan.close()
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(got, ref, mag, dtype, what, tight=False)


def test_odd_feature_dims_of_the_16_bit_types(torch_cuda, hs, oracle):
    """Rows of B and C that start on odd halves.  From three features on the MFMA gather kernels take them: words
    loaded wherever they lie, the lane with the last feature reading one half early and storing one half, and
    beyond 32 features two launches (up to the last multiple of 8; the rest - nine features rather than one).
    Nothing next to C is written.  One feature (matrix times vector): B and C widened to words in a buffer of
    the plan's, two features through the same kernels."""
    torch = torch_cuda
    rng = np.random.default_rng(5)
    for dt in (0, 2):
        for rows, cols, dens, heavy in ((90, 120, 0.1, ()), (300, 3000, 0.004, (5, 100, 299))):
            A = random_csr(rng, rows, cols, dens, dt, 0.2, heavy)
            b = convert(hs, A)
            hs.configure(producer_warp_group_num=16)               # (cut windows: partial sums, second kernel or added inside)
            try:
                plan = hs.Plan(b)
            finally:
                hs.configure()
            for N in (1, 3, 5, 7, 9, 31, 33, 41, 127, 129, 257):
                B = make_b(rng, cols, N, dt)
                ref, mag = oracle_spmm(oracle, A, B, N)
                # C inside a larger buffer of a known pattern: the halves around it must survive
                guard = 64
                buf = torch.full((rows * N + 2 * guard,), 0x7E01, dtype=torch.int16, device="cuda")
                dB = torch.from_numpy(np.ascontiguousarray(B, np.uint16).view(np.int16)).cuda()
                dC = buf[guard:guard + rows * N]
                plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
                torch.cuda.synchronize()
                out = buf.cpu().numpy()
                assert (out[:guard] == 0x7E01).all() and (out[-guard:] == 0x7E01).all(), "N=%d: wrote outside C" % N
                got = out[guard:-guard].reshape(rows, N).view(np.uint16)
                assert_parity(got, ref, mag, dt, "%s odd N=%d" % (DT[dt], N), tight=False)
                # (the denser matrix carries a stream for the LDS-staging kernels, which take any N from 128 on)
                assert plan.info()["last_kernel_family"] == (3 if plan.info()["n_panels"] and N >= 128 else 2)
            got = gpu_spmm(torch_cuda, hs, b, make_b(rng, cols, 34, dt), 34, plan=plan)
            assert plan.info()["last_kernel_family"] == 2
            plan.close()


@pytest.mark.parametrize("dtype", [0, 1])
def test_pointer_alignment_selects_the_kernel_family(torch_cuda, hs, oracle, dtype):
    """B and C need only be aligned to the element size: the LDS-staging kernels load their 16-byte pieces
    wherever they lie and store C element by element, the MFMA gather kernels (kernel mode 3 here) pick their
    load width by the alignment (single words loaded wherever they lie for B or C on an odd half) - with the
    same result (exact integers) whatever the offsets."""
    torch = torch_cuda
    rng = np.random.default_rng(61 + dtype)
    rows, cols, N = 96, 1024, 128
    D = rng.integers(-3, 4, (rows, cols)) * (rng.random((rows, cols)) < 0.2)
    rp = np.zeros(rows + 1, np.uint32)
    ci, vv = [], []
    for r in range(rows):
        nz = np.nonzero(D[r])[0]
        ci += nz.tolist(); vv += D[r, nz].tolist()
        rp[r + 1] = len(ci)
    A = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.array(ci, np.uint32),
             values=encode(np.array(vv, np.float32), dtype))
    plans = {3: hs.Plan(convert(hs, A))}
    assert plans[3].info()["n_panels"] > 0
    hs.set_kernel_mode(3)
    try:
        plans[2] = hs.Plan(convert(hs, A))
    finally:
        hs.set_kernel_mode(0)
    Bm = rng.integers(-4, 5, (cols, N))
    want = encode(D @ Bm, dtype)
    es = 4 if dtype == 1 else 2
    tt = torch.float32 if dtype == 1 else torch.int16
    host_b = torch.from_numpy(encode(Bm, dtype) if dtype == 1 else encode(Bm, dtype).view(np.int16))
    for want_family, off_b, off_c in [(f, b, c) for f in (3, 2) for b, c in ((0, 0), (16, 32), (8, 0), (0, 4), (4, 4), (2, 0), (0, 2), (6, 10))]:
        if off_b % es or off_c % es:
            continue
        plan = plans[want_family]
        buf_b = torch.zeros(cols * N + 16, dtype=tt, device="cuda")
        buf_c = torch.full((rows * N + 16,), 7, dtype=tt, device="cuda")
        dB = buf_b[off_b // es: off_b // es + cols * N]
        dC = buf_c[off_c // es: off_c // es + rows * N]
        dB.copy_(host_b.reshape(-1))
        assert dB.data_ptr() % 16 == off_b % 16 and dC.data_ptr() % 16 == off_c % 16
        plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        got = dC.cpu().numpy().reshape(rows, N)
        got = got if dtype == 1 else got.view(np.uint16)
        assert np.array_equal(got, want), (off_b, off_c)
        # nothing outside C was written
        edge = buf_c.cpu().numpy()
        assert (edge[:off_c // es] == 7).all() and (edge[off_c // es + rows * N:] == 7).all()
        assert plan.info()["last_kernel_family"] == want_family, (off_b, off_c)
    for plan in plans.values():
        plan.close()


def test_matrix_without_entries_gives_zeros(torch_cuda, hs):
    for dt in (0, 1, 2):
        vt = np.float32 if dt == 1 else np.uint16
        b = hs.csr_to_btcf(21, 9, np.zeros(22, np.uint32), np.zeros(0, np.uint32), np.zeros(0, vt), dt)
        plan = hs.Plan(b)
        assert plan.info()["last_kernel_family"] == 0
        for N in (1, 5, 64):
            got = gpu_spmm(torch_cuda, hs, b, np.ones((9, N), vt), N, plan=plan)
            assert got.shape == (21, N) and not got.any()
            assert plan.info()["last_kernel_family"] == 4              # nothing but the clear kernel
        plan.close()


def test_plan_reuse_is_deterministic(torch_cuda, hs, oracle):
    rng = np.random.default_rng(9)
    A = random_csr(rng, 400, 4000, 0.003, 0, 0.1, (3, 200))
    b = convert(hs, A)
    hs.configure(producer_warp_group_num=16)
    try:
        plan = hs.Plan(b)
    finally:
        hs.configure()
    B = make_b(rng, 4000, 128, 0)
    first = gpu_spmm(torch_cuda, hs, b, B, 128, plan=plan)
    # a wider N in between makes the plan regrow its scratch memory
    B2 = make_b(rng, 4000, 512, 0)
    wide = gpu_spmm(torch_cuda, hs, b, B2, 512, plan=plan)
    ref2, mag2 = oracle_spmm(oracle, A, B2, 512)
    assert_parity(wide, ref2, mag2, 0, "N=512 after N=128")
    for _ in range(3):
        again = gpu_spmm(torch_cuda, hs, b, B, 128, plan=plan)
        assert np.array_equal(first, again)           # fixed summation order: bit-identical
    plan.close()


def test_plans_on_different_streams_do_not_disturb_each_other(torch_cuda, hs, oracle):
    """Different plans may run at the same time: each owns its scratch memory.  Three plans
    (cut units with partial sums, the LDS-panel kernel with chunk sums, fp32 storage) are
    launched round robin on three streams without waiting; every output must be bit-identical
    to what the same plan gives alone."""
    torch = torch_cuda
    rng = np.random.default_rng(21)
    cases = []
    for dtype, dens, heavy, N in ((0, 0.003, (3, 200), 64), (2, 0.1, (), 128), (1, 0.1, (), 64)):
        A = random_csr(rng, 400, 4000, dens, dtype, 0.1, heavy)
        b = convert(hs, A)
        hs.configure(producer_warp_group_num=16)
        try:
            plan = hs.Plan(b)
        finally:
            hs.configure()
        B = make_b(rng, 4000, N, dtype)
        alone = gpu_spmm(torch, hs, b, B, N, plan=plan)
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(alone, ref, mag, dtype, "alone, dtype %d" % dtype)
        tt = torch.float32 if dtype == 1 else torch.int16
        dB = torch.from_numpy(B if dtype == 1 else B.view(np.int16)).cuda()
        dC = torch.empty((400, N), dtype=tt, device="cuda")
        cases.append((plan, dB, dC, N, alone, dtype, torch.cuda.Stream()))
    torch.cuda.synchronize()
    for _ in range(20):
        for plan, dB, dC, N, _, _, stream in cases:
            plan.run(dB.data_ptr(), dC.data_ptr(), N, stream.cuda_stream)
    torch.cuda.synchronize()
    for plan, dB, dC, N, alone, dtype, _ in cases:
        got = dC.cpu().numpy()
        got = got if dtype == 1 else got.view(np.uint16)
        assert np.array_equal(got, alone), "dtype %d" % dtype
        plan.close()


@pytest.mark.parametrize("dtype,density,heavy,N", [(0, 0.003, (3, 200, 777), 64), (2, 0.1, (), 256), (1, 0.1, (), 64), (0, 0.02, (5,), 1)])
def test_one_plan_on_several_streams_at_once(torch_cuda, hs, oracle, dtype, density, heavy, N):
    """Launches of one plan on different streams may overlap in time: every stream that launches a plan gets
    partial-sum buffers, arrival counters and (a single feature of a 16-bit type) a vector buffer of its own.
    Three streams, each with its own B and C, launched round robin without waiting; every output must be
    bit-identical to what the plan gives for that B alone, and the plan's device memory grows with the streams."""
    torch = torch_cuda
    rng = np.random.default_rng(31)
    rows, cols = 1600, 8000
    A = random_csr(rng, rows, cols, density, dtype, 0.1, heavy)
    b = convert(hs, A)
    hs.configure(producer_warp_group_num=16)                        # (many ranges: units cut across waves)
    try:
        plan = hs.Plan(b)
    finally:
        hs.configure()
    tt = torch.float32 if dtype == 1 else torch.int16
    lanes = []
    for k in range(3):
        B = make_b(rng, cols, N, dtype)
        alone = gpu_spmm(torch, hs, b, B, N, plan=plan)
        if k == 0:
            ref, mag = oracle_spmm(oracle, A, B, N)
            assert_parity(alone, ref, mag, dtype, "alone")
            assert plan.info()["n_split_windows"] > 0 or plan.info()["n_panels"] > 0    # (something uses the buffers)
        dB = torch.from_numpy(B if dtype == 1 else B.view(np.int16)).cuda()
        dC = torch.empty((rows, N), dtype=tt, device="cuda")
        lanes.append((dB, dC, alone, torch.cuda.Stream()))
    torch.cuda.synchronize()
    one_stream = plan.info()["device_bytes"]
    for _ in range(30):
        for dB, dC, _, stream in lanes:
            plan.run(dB.data_ptr(), dC.data_ptr(), N, stream.cuda_stream)
    torch.cuda.synchronize()
    assert plan.info()["device_bytes"] > one_stream
    for k, (dB, dC, alone, _) in enumerate(lanes):
        got = dC.cpu().numpy()
        got = got if dtype == 1 else got.view(np.uint16)
        assert np.array_equal(got, alone), "stream %d" % k
    plan.close()


def test_run_captured_in_a_hip_graph_replays_correctly(torch_cuda, hs, oracle):
    """After one eager call (which sizes the plan's scratch memory) hspmm_run only
    launches kernels, so a stream capture records it; every replay, with eager work
    and new contents of B in between, must give what the eager call gives."""
    torch = torch_cuda
    rng = np.random.default_rng(15)
    for dtype, panels in ((0, False), (1, False), (0, True), (1, True)):
        if panels:
            # dense windows: the LDS-panel kernel, whose waves add the chunk sums of their units
            A = random_csr(rng, 400, 4000, 0.1, dtype, 0.1)
            b = convert(hs, A)
            plan = hs.Plan(b)
            assert plan.info()["n_panels"] > 0
            N = 128
        else:
            A = random_csr(rng, 400, 4000, 0.003, dtype, 0.1, (3, 200))
            b = convert(hs, A)
            hs.configure(producer_warp_group_num=16)
            try:
                plan = hs.Plan(b)
            finally:
                hs.configure()
            assert plan.info()["n_split_windows"] > 0          # two kernels per call
            N = 64
        tt = torch.int16 if dtype == 0 else torch.float32
        Bs = [make_b(rng, 4000, N, dtype) for _ in range(3)]
        as_t = (lambda x: torch.from_numpy(x.view(np.int16))) if dtype == 0 else torch.from_numpy
        dB = as_t(Bs[0]).cuda()
        dC = torch.empty((400, N), dtype=tt, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            plan.run(dB.data_ptr(), dC.data_ptr(), N, side.cuda_stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
        for rep in range(6):
            Bh = Bs[rep % 3]
            dB.copy_(as_t(Bh).cuda())
            dC.fill_(0x7E01 if dtype == 0 else float("nan"))
            (dB.float().sum() + 1).item()                       # eager work and a synchronisation between replays
            graph.replay()
            torch.cuda.synchronize()
            got = dC.cpu().numpy()
            got = got.view(np.uint16) if dtype == 0 else got
            want = gpu_spmm(torch, hs, b, Bh, N, plan=plan)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "replay %d" % rep
            ref, mag = oracle_spmm(oracle, A, Bh, N)
            assert_parity(got, ref, mag, dtype, "graph replay %d" % rep)
        del graph
        plan.close()


def test_capture_right_after_prepare_on_a_stream_the_plan_has_not_seen(torch_cuda, hs, oracle):
    """hspmm_prepare(plan, N) makes the buffers a stream under capture uses (nothing may be allocated then): the
    first launch of the plan at all may be the one recorded, on a stream of its own, after eager launches on
    another stream as well."""
    torch = torch_cuda
    rng = np.random.default_rng(17)
    for dtype, density, heavy, N, eager_first in ((0, 0.003, (3, 200), 64, False), (1, 0.1, (), 128, False), (2, 0.1, (), 256, True)):
        A = random_csr(rng, 400, 4000, density, dtype, 0.1, heavy)
        b = convert(hs, A)
        hs.configure(producer_warp_group_num=16)
        try:
            plan = hs.Plan(b)
        finally:
            hs.configure()
        B = make_b(rng, 4000, N, dtype)
        tt = torch.float32 if dtype == 1 else torch.int16
        dB = torch.from_numpy(B if dtype == 1 else B.view(np.int16)).cuda()
        dC = torch.empty((400, N), dtype=tt, device="cuda")
        plan.prepare(N)
        if eager_first:
            gpu_spmm(torch, hs, b, B, N, plan=plan)             # (the default stream becomes the plan's first stream)
        before = plan.info()["device_bytes"]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
        assert plan.info()["device_bytes"] == before            # nothing allocated under capture
        want = None
        for rep in range(3):
            dC.fill_(0x7E01 if dtype != 1 else float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = dC.cpu().numpy()
            got = got if dtype == 1 else got.view(np.uint16)
            if want is None:
                want = gpu_spmm(torch, hs, b, B, N, plan=plan)
                ref, mag = oracle_spmm(oracle, A, B, N)
                assert_parity(got, ref, mag, dtype, "recorded launch")
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "replay %d" % rep
        del graph
        plan.close()


def test_graph_captured_at_one_width_survives_launches_at_another(torch_cuda, hs, oracle):
    """A launch recorded in a HIP graph carries the addresses of the plan's partial-sum buffer and
    tables.  Running the same plan eagerly at a wider N afterwards (more partial sums, another number
    of chunks) must leave the recorded launch valid: replays stay bit-identical to the eager result."""
    torch = torch_cuda
    rng = np.random.default_rng(16)
    for dtype, panels in ((0, False), (0, True), (1, True)):
        if panels:
            A = random_csr(rng, 400, 4000, 0.1, dtype, 0.1)
            b = convert(hs, A)
            plan = hs.Plan(b)
            assert plan.info()["n_panels"] > 0
            N1, N2 = 128, 1024
        else:
            A = random_csr(rng, 400, 4000, 0.003, dtype, 0.1, (3, 200))
            b = convert(hs, A)
            hs.configure(producer_warp_group_num=16)
            try:
                plan = hs.Plan(b)
            finally:
                hs.configure()
            assert plan.info()["n_split_windows"] > 0
            N1, N2 = 64, 512
        B1, B2 = make_b(rng, 4000, N1, dtype), make_b(rng, 4000, N2, dtype)
        want1 = gpu_spmm(torch, hs, b, B1, N1, plan=plan)         # eager: sizes the buffers for N1
        tt = torch.int16 if dtype == 0 else torch.float32
        as_t = (lambda x: torch.from_numpy(x.view(np.int16))) if dtype == 0 else torch.from_numpy
        dB = as_t(B1).cuda()
        dC = torch.empty((400, N1), dtype=tt, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            plan.run(dB.data_ptr(), dC.data_ptr(), N1, torch.cuda.current_stream().cuda_stream)
        bytes_before = plan.info()["device_bytes"]
        got2 = gpu_spmm(torch, hs, b, B2, N2, plan=plan)          # a wider launch on the same plan
        assert plan.info()["device_bytes"] > bytes_before, "the wider launch was meant to need more partial sums"
        ref2, mag2 = oracle_spmm(oracle, A, B2, N2)
        assert_parity(got2, ref2, mag2, dtype, "wide launch")
        for rep in range(3):
            dC.fill_(0x7E01 if dtype == 0 else float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = dC.cpu().numpy()
            got = got.view(np.uint16) if dtype == 0 else got
            assert np.array_equal(got.view(np.uint8), want1.view(np.uint8)), "dtype %d panels %s replay %d" % (dtype, panels, rep)
            gpu_spmm(torch, hs, b, B2, N2, plan=plan)             # and again something else in between
        del graph
        plan.close()


def test_bench_entry_point_and_errors(torch_cuda, hs, oracle):
    torch = torch_cuda
    rng = np.random.default_rng(3)
    A = random_csr(rng, 64, 64, 0.2, 0)
    b = convert(hs, A)
    plan = hs.Plan(b)
    B = make_b(rng, 64, 64, 0)
    dB = torch.from_numpy(B.view(np.int16)).cuda()
    dC = torch.zeros((64, 64), dtype=torch.int16, device="cuda")
    ms = plan.bench(dB.data_ptr(), dC.data_ptr(), 64, warmup=3, runs=5)      # src/common.h:48-49
    assert ms > 0
    ref, mag = oracle_spmm(oracle, A, B, 64)
    assert_parity(dC.cpu().numpy().view(np.uint16), ref, mag, 0, "after bench")
    with pytest.raises(hs.HspmmError):
        plan.run(dB.data_ptr(), dC.data_ptr(), 0)                            # N = 0
    with pytest.raises(hs.HspmmError):
        plan.run(0, dC.data_ptr(), 64)                                       # null B
    with pytest.raises(hs.HspmmError):
        plan.run(dB.data_ptr(), 0, 64)                                       # null C
    with pytest.raises(hs.HspmmError):
        plan.bench(dB.data_ptr(), dC.data_ptr(), 64, warmup=0, runs=0)
    info = plan.info()
    assert info["rows"] == 64 and info["compute_units"] > 0 and info["device_bytes"] > 0
    plan.close()


# ------------------------------------------------------------------ the five configurations
@pytest.mark.parametrize("index,shrink", [(0, 1), (1, 8), (2, 64), (3, 8), (4, 8)])
def test_benchmark_configurations_reduced(torch_cuda, hs, oracle, index, shrink):
    from hopper_spmm_amd import generators as G
    cfg = G.make_config(index, shrink)
    A = cfg["A"]
    b = convert(hs, A)
    plan = hs.Plan(b)
    for N in cfg["N"]:
        B = G.dense_b(A["cols"], N, cfg["b_seed"], A["dtype"])
        got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(got, ref, mag, A["dtype"], "%s N=%d" % (cfg["name"], N))
    plan.close()


def _rows_subproblem(A, rows_sel):
    rp = A["row_ptr"].astype(np.int64)
    lens = rp[rows_sel + 1] - rp[rows_sel]
    sub_rp = np.zeros(rows_sel.size + 1, np.uint32)
    sub_rp[1:] = np.cumsum(lens)
    idx = np.concatenate([np.arange(rp[r], rp[r + 1]) for r in rows_sel]) if rows_sel.size else np.zeros(0, np.int64)
    return dict(rows=int(rows_sel.size), cols=A["cols"], dtype=A["dtype"], row_ptr=sub_rp,
                col_idx=A["col_idx"][idx], values=A["values"][idx])


@pytest.mark.parametrize("index,which_n", [(1, 0), (2, 0), (3, 0), (4, 0), (4, 1), (4, 2)])
def test_benchmark_configurations_full_size(torch_cuda, hs, oracle, index, which_n):
    """At full size the oracle is run on a sample of rows only (the heaviest rows
    and a random sample), and size-independent properties cover the rest:
    B = 1 gives the row sums, rows without entries are zero, and the all-shapes
    kernel - an independent implementation - agrees on every element."""
    from hopper_spmm_amd import generators as G
    cfg = G.make_config(index, 1)
    A = cfg["A"]
    dt = A["dtype"]
    b = convert(hs, A)
    N = cfg["N"][which_n]                               # the block-clustered configuration: 16, 64 and 512
    plan = hs.Plan(b)
    B = G.dense_b(A["cols"], N, cfg["b_seed"], dt)
    got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
    if index == 4:
        # N = 16 and 64: gather kernels, one workgroup per unit; N = 512: LDS-panel kernel
        assert plan.info()["last_kernel_family"] == (3 if N == 512 else 2)
    if index == 2:
        # the same matrix handed over as bitmap tiles: they go to the device as they are (no plain tiles on the
        # host, an eighth of the upload) and the gather kernels read the caller's words and elements - same bits
        bm = hs.csr_to_bitmap(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], dt)
        from_bitmap = hs.Plan(bm)
        info = from_bitmap.info()
        assert info["bitmap_from_caller"] == 1 and info["gather_bitmap"] == 1
        assert np.array_equal(gpu_spmm(torch_cuda, hs, bm, B, N, plan=from_bitmap), got)
        from_bitmap.close()
        del bm
    rng = np.random.default_rng(index)
    lens = np.diff(A["row_ptr"].astype(np.int64))
    sel = np.unique(np.concatenate([np.argsort(lens)[-40:], rng.choice(A["rows"], 3000, replace=False)]))
    sub = _rows_subproblem(A, sel)
    ref, mag = oracle_spmm(oracle, sub, B, N)
    assert_parity(got[sel], ref, mag, dt, "%s sampled rows" % cfg["name"])
    assert not got[lens == 0].any()
    # independent implementation on all elements
    hs.set_kernel_mode(1)
    try:
        plan_s = hs.Plan(b)
    finally:
        hs.set_kernel_mode(0)
    other = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan_s)
    plan_s.close()
    if dt == 0:
        assert (half_ulp_distance(got, other) <= 1).mean() > 0.999
        assert np.allclose(got.view(np.float16).astype(np.float32), other.view(np.float16).astype(np.float32),
                           rtol=1e-2, atol=1e-3)
    else:
        assert np.allclose(got, other, rtol=1e-3, atol=1e-4)
    # B = 1: C[r, :] = sum of row r (R-MAT rows sum to 1 by construction)
    ones = np.full((A["cols"], N), 0x3C00, np.uint16) if dt == 0 else np.ones((A["cols"], N), np.float32)
    c1 = gpu_spmm(torch_cuda, hs, b, ones, N, plan=plan)
    vals = A["values"].view(np.float16).astype(np.float64) if dt == 0 else A["values"].astype(np.float64)
    rowsum = np.add.reduceat(np.concatenate([vals, [0.0]]), np.minimum(A["row_ptr"][:-1], vals.size).astype(np.int64))
    rowsum[lens == 0] = 0.0
    absum = np.add.reduceat(np.concatenate([np.abs(vals), [0.0]]), np.minimum(A["row_ptr"][:-1], vals.size).astype(np.int64))
    absum[lens == 0] = 0.0
    c1f = c1.view(np.float16).astype(np.float64) if dt == 0 else c1.astype(np.float64)
    tol = (2e-3 if dt == 0 else 1e-5) * np.abs(rowsum) + 1e-5 * absum + 1e-7
    assert np.all(np.abs(c1f - rowsum[:, None]) <= tol[:, None])
    assert np.all(c1f == c1f[:, :1])                     # every feature column identical
    plan.close()


def test_more_than_2_to_24_tiles_and_4_gib_of_tiles_and_of_output(torch_cuda, hs):
    """Sizes past the 24- and 32-bit marks: 8.4 M windows of two tiles each (16.8 M tiles, 4.3 GB of them) over
    67 M rows (4.3 GB of C at N = 32).  Small integers, so every sum is exact: the default kernels must agree bit
    for bit with the all-shapes kernel on every output and with numpy on sampled rows."""
    torch = torch_cuda
    W, N, cols = (1 << 23) + 4096, 32, 4096
    rows = W * 8
    per_row = np.array([3, 2, 2, 2, 2, 2, 2, 2], np.int64)           # 17 distinct columns per window
    row_ptr = np.zeros(rows + 1, np.uint32)
    row_ptr[1:] = np.cumsum(np.tile(per_row, W))
    nnz = int(row_ptr[-1])
    rng = np.random.default_rng(1)
    first = rng.integers(0, cols - 37 * 17, W).astype(np.uint32)
    order = np.array([0, 8, 16, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15], np.uint32)   # a window's entries row by row
    col_idx = (first[:, None] + 37 * order[None, :]).astype(np.uint32).reshape(-1)
    vals = rng.integers(-3, 4, nnz).astype(np.float16)
    b = hs.csr_to_btcf(rows, cols, row_ptr, col_idx, vals.view(np.uint16), 0)
    assert b["total_tiles"] > 1 << 24 and b["data"].nbytes > 1 << 32
    B = rng.integers(-4, 5, (cols, N)).astype(np.float16)
    dB = torch.from_numpy(B.view(np.int16)).cuda()
    outs = []
    for mode in (0, 1):
        hs.set_kernel_mode(mode)
        try:
            plan = hs.Plan(b)
        finally:
            hs.set_kernel_mode(0)
        dC = torch.empty((rows, N), dtype=torch.int16, device="cuda")
        dC.fill_(0x7E01)
        plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert plan.info()["last_kernel_family"] == (2 if mode == 0 else 1)
        plan.close()
        outs.append(dC)
    assert outs[0].numel() * 2 > 1 << 32
    assert torch.equal(outs[0], outs[1])
    sample = np.unique(np.concatenate([np.arange(64), np.arange(rows - 64, rows), np.arange(rows // 2 - 32, rows // 2 + 32),
                                       rng.integers(0, rows, 2000)]))
    got = outs[0][torch.from_numpy(sample).cuda()].cpu().numpy().view(np.float16).astype(np.float32)
    av, Bf = vals.astype(np.float32), B.astype(np.float32)
    for i, r in enumerate(sample):
        lo, hi = int(row_ptr[r]), int(row_ptr[r + 1])
        assert np.array_equal((av[lo:hi, None] * Bf[col_idx[lo:hi]]).sum(0), got[i]), "row %d" % r
    del outs, dC, dB
    torch.cuda.empty_cache()


def test_lds_panel_stream_of_more_than_4_gib(torch_cuda, hs):
    """65536 x 32768 at 10 %, fp32 storage: 3.7 M steps of 2 KB in the stream of the LDS-staging kernels (7.5 GB, past
    32-bit byte offsets), 19 M tiles from the caller.  Small integers (exact in bf16 parts and in fp32 sums): bit for
    bit against the all-shapes kernel."""
    torch = torch_cuda
    rows, cols, N, mean_gap = 65536, 32768, 64, 10
    rng = np.random.default_rng(2)
    per = cols // mean_gap + cols // (mean_gap * 8) + 16
    counts, chunks = np.zeros(rows + 1, np.int64), []
    for r0 in range(0, rows, 4096):
        gaps = rng.integers(1, 2 * mean_gap, (4096, per), dtype=np.int32)         # ascending columns, 10 apart on average
        gaps[:, 0] = rng.integers(0, mean_gap, 4096)
        c = np.cumsum(gaps, axis=1, dtype=np.int32)
        keep = c < cols
        counts[r0 + 1:r0 + 4097] = keep.sum(1)
        chunks.append(c[keep].astype(np.uint32))
    col_idx = np.concatenate(chunks)
    del chunks
    row_ptr = np.cumsum(counts).astype(np.uint32)
    vals = rng.integers(-3, 4, int(row_ptr[-1])).astype(np.float32)
    b = hs.csr_to_btcf(rows, cols, row_ptr, col_idx, vals, 1)
    dB = torch.from_numpy(rng.integers(-4, 5, (cols, N)).astype(np.float32)).cuda()
    outs = []
    for mode in (0, 1):
        hs.set_kernel_mode(mode)
        try:
            plan = hs.Plan(b)
        finally:
            hs.set_kernel_mode(0)
        dC = torch.full((rows, N), float("nan"), dtype=torch.float32, device="cuda")
        plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        info = plan.info()
        assert info["last_kernel_family"] == (3 if mode == 0 else 1)
        if mode == 0:
            assert info["n_panel_steps"] * 2048 > 1 << 32
        plan.close()
        outs.append(dC)
    assert torch.equal(outs[0].view(torch.int32), outs[1].view(torch.int32))
    del outs, dC, dB
    torch.cuda.empty_cache()


def test_columns_beyond_the_32_bit_offset_range(torch_cuda, hs, oracle):
    """B larger than 4 GiB: the gather uses 64-bit addresses."""
    torch = torch_cuda
    cols, N = (1 << 24) + 96, 128
    rng = np.random.default_rng(12)
    used = np.unique(np.concatenate([rng.choice(cols, 300, replace=False), [0, cols - 1, (1 << 24) - 1, 1 << 24]]))
    rows = 40
    rl = [np.sort(rng.choice(used, int(rng.integers(0, 30)), replace=False)).astype(np.uint32) for _ in range(rows)]
    rp = np.zeros(rows + 1, np.uint32)
    rp[1:] = np.cumsum([len(x) for x in rl])
    ci = np.concatenate(rl).astype(np.uint32)
    vals = rng.uniform(-1, 1, ci.size).astype(np.float32).astype(np.float16).view(np.uint16)
    b = hs.csr_to_btcf(rows, cols, rp, ci, vals, 0)
    small = make_b(rng, used.size, N, 0)                 # B rows that are referenced
    dB = torch.zeros((cols, N), dtype=torch.int16, device="cuda")
    dB[torch.from_numpy(used.astype(np.int64)).cuda()] = torch.from_numpy(small.view(np.int16)).cuda()
    dC = torch.empty((rows, N), dtype=torch.int16, device="cuda")
    plan = hs.Plan(b)
    plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = dC.cpu().numpy().view(np.uint16)
    plan.close()
    remap = np.searchsorted(used, ci).astype(np.uint32)
    ref, mag = oracle.spmm_csr_f16(rows, N, rp, remap, vals, small, want_absdot=True)
    assert_parity(got, ref, mag, 0, "wide B")


# ------------------------------------------------------------------ feature blocks with XCDs of their own
@pytest.mark.parametrize("dtype", [0, 2])
def test_feature_blocks_dealt_out_by_xcd(torch_cuda, hs, oracle, dtype):
    """The gather kernels can give each of 2, 4 or 8 feature blocks XCDs of its own (every L2 then
    caches one part of each B row only).  Forced on here for a small matrix: the work numbering
    must still cover every range and every feature block, with and without cut units."""
    rng = np.random.default_rng(40 + dtype)
    A = random_csr(rng, 700, 900, 0.03, dtype, heavy_rows=(5, 333))
    b = convert(hs, A)
    for N in (128, 256, 512):
        B = make_b(rng, A["cols"], N, dtype)
        ref, mag = oracle_spmm(oracle, A, B, N)
        results = []
        for split in ("0", "1"):
            os.environ["HSPMM_XCD_SPLIT"] = split
            try:
                hs.set_kernel_mode(3)
                plan = hs.Plan(b)
            finally:
                hs.set_kernel_mode(0)
                os.environ.pop("HSPMM_XCD_SPLIT", None)
            got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
            assert plan.info()["last_kernel_family"] == 2
            plan.close()
            assert_parity(got, ref, mag, dtype, "XCD split %s N=%d" % (split, N))
            results.append(got)
    # exact-integer inputs: bit-exact whatever the numbering
    rows, cols = 300, 500
    D = rng.integers(-3, 4, (rows, cols)) * (rng.random((rows, cols)) < 0.05)
    rr, cc = np.nonzero(D)
    rp = np.zeros(rows + 1, np.uint32)
    rp[1:] = np.cumsum(np.bincount(rr, minlength=rows))
    Ai = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=cc.astype(np.uint32),
              values=encode(D[rr, cc].astype(np.float32), dtype))
    bi = convert(hs, Ai)
    Bm = rng.integers(-4, 5, (cols, 128))
    os.environ["HSPMM_XCD_SPLIT"] = "1"
    try:
        plan = hs.Plan(bi)
    finally:
        os.environ.pop("HSPMM_XCD_SPLIT", None)
    got = gpu_spmm(torch_cuda, hs, bi, encode(Bm, dtype), 128, plan=plan)
    plan.close()
    assert np.array_equal(got, encode(D @ Bm, dtype))


# ------------------------------------------------------------------ bitmap tiles on the device
@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_panel_stream_with_two_units_per_wave_and_packed_tiles(torch_cuda, hs, oracle, dtype):
    """hspmm_set_panel_stream: 1 = every consumer wave of the LDS-staging kernels takes two units,
    2 = also the tiles of the steps without their zeros (masks + stored values, expanded in
    registers).  The MFMA inputs are the same in all three modes, so with the same split into
    chunks of panels the results are bit-identical; and exact-integer inputs are exact."""
    if not hs.has_experimental():
        with pytest.raises(hs.HspmmError) as e:            # refused with a message, not ignored
            hs.set_panel_stream(1)
        assert e.value.code == 5 and "EXPERIMENTAL" in str(e.value)
        pytest.skip("stream modes 1 and 2 of the LDS-staging kernels exist in libraries built with EXPERIMENTAL=1 only")
    rng = np.random.default_rng(70 + dtype)
    feature_dims = (64, 128) if dtype == 1 else (128, 384)
    cases = [
        random_csr(rng, 300, 1000, 0.1, dtype, empty_row_prob=0.05),          # unions of overlapping column lists
        random_csr(rng, 77, 530, 0.3, dtype),                                  # odd number of units, ragged last window
        random_csr(rng, 24, 3000, 0.02, dtype, heavy_rows=(3,)),               # three windows, long runs of empty panels
    ]
    hs.set_kernel_mode(4)
    try:
        for ci, A in enumerate(cases):
            b = convert(hs, A)
            for N in feature_dims:
                B = make_b(rng, A["cols"], N, dtype)
                ref, mag = oracle_spmm(oracle, A, B, N)
                for chunks in ("1", "3"):
                    os.environ["HSPMM_PANEL_CHUNKS"] = chunks
                    got = {}
                    try:
                        for mode in (0, 1, 2):
                            hs.set_panel_stream(mode)
                            plan = hs.Plan(b)
                            got[mode] = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
                            info = plan.info()
                            plan.close()
                            assert info["last_kernel_family"] == 3
                            assert info["panel_stream_mode"] == mode, (ci, N, mode, info)
                    finally:
                        hs.set_panel_stream(0)
                        os.environ.pop("HSPMM_PANEL_CHUNKS", None)
                    assert_parity(got[0], ref, mag, dtype, "case %d N=%d chunks=%s" % (ci, N, chunks))
                    assert np.array_equal(got[1], got[0]), "two units per wave: case %d N=%d chunks=%s" % (ci, N, chunks)
                    assert np.array_equal(got[2], got[0]), "packed tiles: case %d N=%d chunks=%s" % (ci, N, chunks)
        # exact integers, with stored zeros, negative zeros and a dense window among sparse ones
        rows, cols = 90, 700
        D = rng.integers(-3, 4, (rows, cols)) * (rng.random((rows, cols)) < 0.12)
        D[16:24] = rng.integers(1, 4, (8, cols))
        rr, cc = np.nonzero(D)
        rp = np.zeros(rows + 1, np.uint32)
        rp[1:] = np.cumsum(np.bincount(rr, minlength=rows))
        vals = D[rr, cc].astype(np.float32)
        vals[::17] = 0.0                                                        # stored zeros
        vals[5::29] = -0.0
        D2 = np.zeros((rows, cols))
        D2[rr, cc] = vals
        Ai = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=cc.astype(np.uint32), values=encode(vals, dtype))
        bi = convert(hs, Ai)
        N = feature_dims[0]
        Bm = rng.integers(-4, 5, (cols, N))
        for mode in (1, 2):
            hs.set_panel_stream(mode)
            plan = hs.Plan(bi)
            got = gpu_spmm(torch_cuda, hs, bi, encode(Bm, dtype), N, plan=plan)
            assert plan.info()["panel_stream_mode"] == mode
            plan.close()
            # (the sums are exact in fp32; the output is their one rounding to the storage type)
            assert np.array_equal(decode(got, dtype), decode(encode(D2 @ Bm, dtype), dtype)), "mode %d" % mode
        # A wave's second unit whose first step lies more than 15 panels behind the first unit's last one (the
        # steps count the panels from their predecessor in four bits): single windows, 36 panels, the second
        # window's only columns in panel 30.
        rows, cols = 32, 9000
        D = np.zeros((rows, cols))
        D[0, 3] = 2; D[1, 200] = -1                     # window 0: panel 0
        D[8, 7700] = 3; D[9, 7701] = 1                  # window 1: panel 30 only
        D[16, 5000] = 1; D[17, 8999] = -2               # window 2: panels 19 and 35
        D[24, 100] = 1                                  # window 3: panel 0 (and an odd man out when units are paired up)
        rr, cc = np.nonzero(D)
        rp = np.zeros(rows + 1, np.uint32)
        rp[1:] = np.cumsum(np.bincount(rr, minlength=rows))
        Af = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=cc.astype(np.uint32), values=encode(D[rr, cc].astype(np.float32), dtype))
        bf = convert(hs, Af)
        Bm = rng.integers(-4, 5, (cols, N))
        hs.set_window_pairing(1)                        # (single windows stay single)
        try:
            for mode in (0, 1, 2):
                hs.set_panel_stream(mode)
                plan = hs.Plan(bf)
                got = gpu_spmm(torch_cuda, hs, bf, encode(Bm, dtype), N, plan=plan)
                assert plan.info()["panel_stream_mode"] == mode and plan.info()["last_kernel_family"] == 3
                plan.close()
                assert np.array_equal(decode(got, dtype), decode(encode(D @ Bm, dtype), dtype)), "far first step, mode %d" % mode
        finally:
            hs.set_window_pairing(0)
    finally:
        hs.set_panel_stream(0)
        hs.set_kernel_mode(0)


# ------------------------------------------------------------------ staging layout of the LDS-panel kernels
@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_lds_staging_hands_every_b_row_to_its_column(torch_cuda, hs, dtype):
    """The LDS-staging kernels copy rows of B into an LDS image and read them back with the
    transposing LDS read (the row gathered by the address, four k of one feature per lane).  Here every
    row of A has a single entry 1 at column c, and B[k][f] encodes (k, f): row r of C must be row c of
    B, bit for bit.  The entry visits every k-slot of a 32-column step, both windows of a pair of
    windows, columns in several panels and both LDS images (the reference checks its staged copy the
    same way, by coordinates: test/01.tma_copy_matrix/copy.cu:149-170)."""
    rng = np.random.default_rng(90 + dtype)
    rows, cols, N = 16, 700, 128 if dtype != 1 else 64
    k_idx, f_idx = np.meshgrid(np.arange(cols), np.arange(N), indexing="ij")
    Bm = (k_idx * 5 + f_idx * 3) % 251                                   # exact in every element type; rows differ
    B = encode(Bm.astype(np.float32), dtype)
    # 40 columns: a full step of 32 in panel 0, some in panel 1 (256..511) and panel 2
    used = np.sort(np.concatenate([rng.choice(256, 32, replace=False), 256 + rng.choice(256, 5, replace=False),
                                   512 + rng.choice(188, 3, replace=False)])).astype(np.uint32)
    hs.set_kernel_mode(4)
    try:
        for shift in range(used.size):
            # every used column appears (so that the window's column list, and the step layout, stay the same)
            # with value 0, except the one per row that carries the 1
            hot = used[(np.arange(rows) * 3 + shift) % used.size]
            vals = np.zeros((rows, used.size), np.float32)
            vals[np.arange(rows), (np.arange(rows) * 3 + shift) % used.size] = 1.0
            rp = (np.arange(rows + 1) * used.size).astype(np.uint32)
            A = dict(rows=rows, cols=cols, dtype=dtype, row_ptr=rp, col_idx=np.tile(used, rows),
                     values=encode(vals.reshape(-1), dtype))
            b = convert(hs, A)
            plan = hs.Plan(b)
            got = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
            assert plan.info()["last_kernel_family"] == 3
            plan.close()
            want = decode(B, dtype)[hot]
            assert np.array_equal(decode(got, dtype), want), "shift %d" % shift
    finally:
        hs.set_kernel_mode(0)


# ------------------------------------------------------------------ bitmap tiles in the gather kernels
@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_gather_kernels_read_bitmap_tiles(torch_cuda, hs, oracle, dtype):
    """Single windows with few stored elements per tile are kept on the device as the reference's bitmap
    tiles (128 bits per 8 x 16 tile, 64 per 8 x 8 tile of fp32 storage, + the stored elements) and expanded in
    registers by the gather kernels.  The MFMA inputs are those of the uncompressed tiles, so the results are
    bit-identical; stored zeros, negative zeros, full tiles and tiles with one element are all in here."""
    rng = np.random.default_rng(120 + dtype)
    rows, cols = 530, 1500
    A = random_csr(rng, rows, cols, 0.01, dtype, empty_row_prob=0.1, heavy_rows=(7, 300))
    v = decode(A["values"], dtype).astype(np.float32)
    v[::13] = 0.0                                    # stored zeros (not kept by the bitmap: +0 is "not stored")
    v[3::31] = -0.0                                  # negative zeros are
    A["values"] = encode(v, dtype)
    b = convert(hs, A)
    # (fp32 storage: every width of the lanes' loads - 1, 2, 4 words - has a bitmap form; kernel mode 3 keeps
    # the plan off the LDS-staging kernels, which fp32 storage prefers from this density on)
    for N in (64, 128, 256, 512) if dtype != 1 else (8, 16, 24, 32, 64, 128, 256):
        B = make_b(rng, cols, N, dtype)
        ref, mag = oracle_spmm(oracle, A, B, N)
        got = {}
        for use in ("0", "1"):
            os.environ["HSPMM_GATHER_BITMAP"] = use
            hs.set_kernel_mode(3 if dtype == 1 else 0)
            try:
                plan = hs.Plan(b)
                got[use] = gpu_spmm(torch_cuda, hs, b, B, N, plan=plan)
            finally:
                hs.set_kernel_mode(0)
                os.environ.pop("HSPMM_GATHER_BITMAP", None)
            info = plan.info()
            plan.close()
            assert info["last_kernel_family"] == 2 and info["gather_bitmap"] == int(use)
        hs.set_kernel_mode(3 if dtype == 1 else 0)       # (the tolerance of fp32 storage depends on the kernels in use)
        try:
            assert_parity(got["0"], ref, mag, dtype, "tiles N=%d" % N)
        finally:
            hs.set_kernel_mode(0)
        assert np.array_equal(got["1"].view(np.uint8), got["0"].view(np.uint8)), "bitmap tiles differ at N=%d" % N
    # dense 8 x 16 tiles (every bit set) next to empty windows, forced through the bitmap path
    D = np.zeros((64, 96))
    D[0:8, 0:16] = rng.integers(1, 4, (8, 16))
    D[8:16, 5:85] = rng.integers(-3, 4, (8, 80))
    D[40, 95] = 2
    rr, cc = np.nonzero(D)
    rp = np.zeros(65, np.uint32)
    rp[1:] = np.cumsum(np.bincount(rr, minlength=64))
    Ai = dict(rows=64, cols=96, dtype=dtype, row_ptr=rp, col_idx=cc.astype(np.uint32), values=encode(D[rr, cc].astype(np.float32), dtype))
    Bm = rng.integers(-4, 5, (96, 128))
    os.environ["HSPMM_GATHER_BITMAP"] = "1"
    hs.set_kernel_mode(3)                            # (dense windows: keep the plan off the LDS-staging kernels)
    try:
        plan = hs.Plan(convert(hs, Ai))
    finally:
        hs.set_kernel_mode(0)
        os.environ.pop("HSPMM_GATHER_BITMAP", None)
    got = gpu_spmm(torch_cuda, hs, convert(hs, Ai), encode(Bm, dtype), 128, plan=plan)
    assert plan.info()["gather_bitmap"] == 1 and plan.info()["last_kernel_family"] == 2
    plan.close()
    assert np.array_equal(decode(got, dtype), decode(encode(D @ Bm, dtype), dtype))
