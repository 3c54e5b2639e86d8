"""The command-line drivers fp16_test / tf32_test (arguments of the reference's
main, reference src/fp16.cu:283-319)."""
import os
import subprocess

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def run(hs, name, *args):
    exe = hs.cli_path(name)
    assert os.path.exists(exe), "build the drivers first (hopper_spmm_amd.build_library)"
    return subprocess.run([exe, *args], capture_output=True, text=True, timeout=120)


def test_usage_and_bad_arguments(hs):
    for name in ("fp16_test", "tf32_test"):
        r = run(hs, name)
        assert r.returncode == 1 and "Usage" in r.stdout            # src/fp16.cu:285-288
        r = run(hs, name, os.path.join(GOLD, "tiny.mtx"), "0")
        assert r.returncode == 1
        r = run(hs, name, "/nonexistent/file.mtx", "8")
        assert r.returncode == 1 and "cannot open" in r.stdout       # src/utils/load.h:176-180


def test_cli_fails_loudly_without_a_device(hs):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    r = run(hs, "fp16_test", os.path.join(GOLD, "tiny.mtx"), "64")
    assert r.returncode == 1 and "hspmm_create" in r.stderr
    assert "tiles (8 x 16): 2" in r.stdout                           # the format statistics of src/fp16.cu:295-301
    for fmt, entry in (("bitmap", "hspmm_create_bitmap"), ("grouped", "hspmm_create_grouped"),
                       ("balanced", "hspmm_create_bitmap")):
        r = run(hs, "fp16_test", os.path.join(GOLD, "tiny.mtx"), "64", "--format", fmt)
        assert r.returncode == 1 and entry in r.stderr
        assert "2 tiles, 9 stored entries" in r.stdout
    r = run(hs, "fp16_test", os.path.join(GOLD, "tiny.mtx"), "64", "--format", "csr")
    assert r.returncode == 1 and "unknown format" in r.stdout


@pytest.mark.gpu
def test_cli_end_to_end_with_verification(hs, tmp_path):
    rng = np.random.default_rng(8)
    rows, cols, nnz = 500, 700, 6000
    flat = rng.choice(rows * cols, nnz, replace=False)
    p = tmp_path / "m.mtx"
    with open(p, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n%d %d %d\n" % (rows, cols, nnz))
        for k in flat:
            f.write("%d %d %.6g\n" % (k // cols + 1, k % cols + 1, rng.normal()))
    for name, n, fmt in (("fp16_test", "128", "tiles"), ("fp16_test", "7", "tiles"), ("tf32_test", "64", "tiles"),
                         ("bf16_test", "128", "tiles"), ("bf16_test", "5", "tiles"), ("fp16_test", "64", "bitmap"),
                         ("tf32_test", "32", "grouped"), ("bf16_test", "64", "grouped"),
                         ("fp16_test", "64", "balanced"), ("tf32_test", "16", "balanced"),
                         # tiles written column by column (-DSPARSE_A_TRANSPOSE)
                         ("fp16_transposed_test", "128", "tiles"), ("fp16_transposed_test", "40", "bitmap"),
                         # the tf32 variant with 8 x 4 tiles (-DMMA_M16N8K4, reference src/common.h:28-35)
                         ("tf32_k4_test", "64", "tiles"), ("tf32_k4_test", "7", "tiles")):
        r = run(hs, name, str(p), n, "--seed", "42", "--verify", "--format", fmt)
        assert r.returncode == 0, r.stdout + r.stderr
        assert "verification passed" in r.stdout
        assert "SpMM timed runs: 5" in r.stdout                      # RUNS, src/common.h:49
        assert "stored entries: %d" % nnz in r.stdout


@pytest.mark.gpu
def test_cli_balanced_groups_of_a_block_clustered_matrix(hs, tmp_path):
    """--format balanced on a matrix whose adjacent windows share their column lists (16 x 16 blocks): the plan
    behind BTCF2GBTCF_balanced pairs those windows, and still hands out groups of the caller's tiles."""
    rng = np.random.default_rng(9)
    rows, cols = 256, 640
    p = tmp_path / "blocks.mtx"
    entries = []
    for bi in range(0, rows, 16):
        for bj in range(0, cols, 16):
            if rng.random() < 0.5:
                for r in range(16):
                    for c in range(16):
                        entries.append((bi + r + 1, bj + c + 1, rng.normal()))
    with open(p, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n%d %d %d\n" % (rows, cols, len(entries)))
        for r, c, v in entries:
            f.write("%d %d %.6g\n" % (r, c, v))
    for name in ("fp16_test", "tf32_test"):
        r = run(hs, name, str(p), "64", "--seed", "7", "--verify", "--format", "balanced")
        assert r.returncode == 0, r.stdout + r.stderr
        assert "verification passed" in r.stdout and "total groups" in r.stdout
