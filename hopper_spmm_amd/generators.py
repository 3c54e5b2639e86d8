"""Deterministic synthetic inputs for the benchmark configurations.

The reference ships no matrices (its `matrix/` directory is git-ignored,
reference .gitignore:2) and fills B with unseeded rand() (reference
src/fp16.cu:303-309).  These generators build matrices of the named shapes from
fixed seeds, always without duplicate (row, column) entries, because the
reference's format conversion overwrites duplicates instead of summing them
(reference src/utils/convert.h:215).

Random numbers: the raw 64-bit words of the counter-based Philox 4x64-10 generator
(numpy's bit generator, whose stream numpy keeps stable across versions and
platforms) turned into uniforms, bounded integers and normals by the transforms
of `Stream` below - none of numpy's distribution methods, which may change from
one numpy version to the next.  tests/test_generators.py pins digests of the
generated matrices.

All matrices are returned in CSR form as produced by the reference's loader
(reference src/utils/load.h:281-300): rows ascending, columns ascending inside
a row.  fp16 values are returned as uint16 bit patterns (round to nearest even).
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

FP16, TF32, BF16 = 0, 1, 2
_CHUNK = 1 << 18          # pairs of normals per task of Stream.normal32


class Stream:
    """Uniforms, bounded integers and normals from the raw words of Philox(seed), in the order they are asked for."""

    def __init__(self, seed):
        self.bits = np.random.Philox(int(seed))

    def words32(self, n):
        """n 32-bit words: the low, then the high half of every 64-bit word (an odd n leaves a half unused)."""
        raw = self.bits.random_raw((int(n) + 1) // 2)
        return np.atleast_1d(raw).astype("<u8").view("<u4")[:int(n)]

    def uniform32(self, shape):
        """float32 in [0, 1): the top 24 bits of a 32-bit word."""
        n = int(np.prod(shape))
        return ((self.words32(n) >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)).reshape(shape)

    def uniform64(self, low, high, n):
        """float64 in [low, high): the top 53 bits of a 64-bit word."""
        raw = np.atleast_1d(self.bits.random_raw(int(n)))
        return low + (high - low) * ((raw >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0))

    def below(self, bound, n):
        """int64 in [0, bound), bound <= 2^32: the high word of a 32-bit word times bound (exactly uniform when
        bound is a power of two, which is what the configurations use; else biased by < bound / 2^32)."""
        return ((self.words32(n).astype(np.uint64) * np.uint64(bound)) >> np.uint64(32)).astype(np.int64)

    def normal32(self, shape):
        """Standard normals as float32, Box-Muller in float64 on two words per pair of values:
        sqrt(-2 ln u1) (cos, sin)(2 pi u2), u1 in (0, 1], u2 in [0, 1)."""
        n = int(np.prod(shape))
        pairs = (n + 1) // 2
        raw = np.atleast_1d(self.bits.random_raw(2 * pairs)).reshape(pairs, 2)
        out = np.empty((pairs, 2), np.float32)

        def transform(first):
            part = raw[first:first + _CHUNK]
            u1 = ((part[:, 0] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
            u2 = (part[:, 1] >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
            radius = np.sqrt(-2.0 * np.log(u1))
            out[first:first + _CHUNK, 0] = radius * np.cos(2.0 * np.pi * u2)
            out[first:first + _CHUNK, 1] = radius * np.sin(2.0 * np.pi * u2)

        # (numpy's element-wise loops run without the interpreter lock: the chunks go to threads; every value
        # depends on its own two words only, so the result does not depend on the number of threads)
        firsts = range(0, pairs, _CHUNK)
        if len(firsts) > 1:
            with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as pool:
                list(pool.map(transform, firsts))
        else:
            transform(0)
        return out.reshape(-1)[:n].reshape(shape)


def _rng(seed):
    return Stream(seed)


def half_bits(x):
    """float array -> IEEE half bit patterns (uint16), round to nearest even."""
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16)


def bf16_bits(x):
    """float array -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(np.asarray(x, np.float32))
    if nan.any():
        r = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
    return r


def encode(x, dtype):
    """float values -> the storage of `dtype` (uint16 bits for fp16 / bf16, float32 otherwise)."""
    if dtype == FP16:
        return half_bits(x)
    if dtype == BF16:
        return bf16_bits(x)
    return np.asarray(x, np.float32)


def csr_from_keys(rows, cols, keys, values_fn, dtype):
    """keys: sorted unique int64 array of row * cols + col."""
    r = (keys // cols).astype(np.int64)
    c = (keys % cols).astype(np.uint32)
    counts = np.bincount(r, minlength=rows)
    row_ptr = np.zeros(rows + 1, np.uint32)
    np.cumsum(counts, out=row_ptr[1:])
    vals = values_fn(r, c, counts)
    vals = encode(vals, dtype)
    return dict(rows=int(rows), cols=int(cols), nnzs=int(keys.size), dtype=dtype,
                row_ptr=row_ptr, col_idx=c, values=vals)


def uniform_mask(rows, cols, density, seed, dtype=FP16):
    """Bernoulli(density) mask, values U(-1, 1) (configuration 1)."""
    g = _rng(seed)
    parts = []
    step = max(1, (1 << 24) // max(cols, 1))
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        m = g.uniform32((r1 - r0, cols)) < density
        rr, cc = np.nonzero(m)
        parts.append((rr.astype(np.int64) + r0) * cols + cc)
    keys = np.concatenate(parts) if parts else np.zeros(0, np.int64)
    return csr_from_keys(rows, cols, keys, lambda r, c, n: g.uniform64(-1.0, 1.0, r.size).astype(np.float32), dtype)


def uniform_draws(rows, cols, draws_per_row, seed, dtype=FP16):
    """rows * draws_per_row uniform (row, col) draws, duplicates removed, values
    U(-1, 1) (configuration 2)."""
    g = _rng(seed)
    n = int(rows) * int(draws_per_row)
    r = g.below(rows, n)
    c = g.below(cols, n)
    keys = np.unique(r * cols + c)
    return csr_from_keys(rows, cols, keys, lambda r, c, n: g.uniform64(-1.0, 1.0, r.size).astype(np.float32), dtype)


def rmat(scale, edge_factor, seed, a=0.57, b=0.19, c=0.19, d=0.05, dtype=FP16):
    """R-MAT power-law adjacency: 2^scale vertices, edge_factor * 2^scale edge
    draws with quadrant probabilities (a, b, c, d), duplicates removed, no vertex
    permutation, value(i, j) = 1 / out-degree(i) (configuration 3)."""
    g = _rng(seed)
    nv = 1 << scale
    ne = int(edge_factor) * nv
    r = np.zeros(ne, np.int64)
    col = np.zeros(ne, np.int64)
    ab, abc = a + b, a + b + c
    for _ in range(scale):
        u = g.uniform32(ne)
        rbit = u >= ab                      # quadrants c, d: lower half
        cbit = ((u >= a) & (u < ab)) | (u >= abc)   # quadrants b, d: right half
        r = (r << 1) | rbit
        col = (col << 1) | cbit
    keys = np.unique(r * nv + col)
    return csr_from_keys(nv, nv, keys, lambda r, c, n: (1.0 / n[r]).astype(np.float32), dtype)


def pruned_weight(rows, cols, keep_fraction, seed, std=0.02, dtype=TF32):
    """Dense N(0, std) weight, the keep_fraction largest magnitudes kept
    (magnitude pruning, configuration 4)."""
    g = _rng(seed)
    w = g.normal32((rows, cols)) * np.float32(std)
    k = int(round(rows * cols * keep_fraction))
    flat = np.abs(w).ravel()
    if k <= 0:
        keys = np.zeros(0, np.int64)
    else:
        thr = np.partition(flat, flat.size - k)[flat.size - k]
        keys = np.nonzero(flat >= thr)[0].astype(np.int64)
    wf = w.ravel()
    return csr_from_keys(rows, cols, keys, lambda r, c, n: wf[r * cols + c], dtype)


def block_sparse(rows, cols, block, keep_probability, seed, std=0.02, dtype=FP16):
    """Nonzeros clustered in block x block squares kept with keep_probability,
    values N(0, std) (configuration 5)."""
    g = _rng(seed)
    br, bc = (rows + block - 1) // block, (cols + block - 1) // block
    keep = g.uniform32((br, bc)) < keep_probability
    bi, bj = np.nonzero(keep)
    ii, jj = np.meshgrid(np.arange(block), np.arange(block), indexing="ij")
    r = (bi[:, None, None] * block + ii[None]).reshape(-1).astype(np.int64)
    c = (bj[:, None, None] * block + jj[None]).reshape(-1).astype(np.int64)
    ok = (r < rows) & (c < cols)
    keys = np.sort(r[ok] * cols + c[ok])
    return csr_from_keys(rows, cols, keys,
                         lambda r, c, n: g.normal32(r.size) * np.float32(std), dtype)


def dense_b(cols, N, seed, dtype=FP16):
    """B = N(0, 1), row-major cols x N; uint16 half bits for fp16, float32 otherwise."""
    g = _rng(seed)
    x = g.normal32((cols, N))
    return encode(x, dtype)


# The five configurations the benchmark names; `shrink` divides the sizes for
# tests (1 = full size).  N is a tuple for the batch sweep of configuration 5.
def make_config(index, shrink=1, seed=None):
    s = int(shrink)
    if index == 0:
        n = 4096 // s
        A = uniform_mask(n, n, 0.01, 1001 if seed is None else seed)
        return dict(name="uniform 1%% %dx%d fp16" % (n, n), A=A, N=(64,), b_seed=2001)
    if index == 1:
        n = 65536 // s
        A = uniform_draws(n, n, 16, 1002 if seed is None else seed)
        return dict(name="uniform ~16/row %dx%d fp16" % (n, n), A=A, N=(128,), b_seed=2002)
    if index == 2:
        scale = 20
        while s > 1:
            scale -= 1
            s //= 2
        A = rmat(scale, 16, 1003 if seed is None else seed)
        return dict(name="R-MAT scale %d deg 16 fp16" % scale, A=A, N=(128,), b_seed=2003)
    if index == 3:
        r, c = 11008 // s, 4096 // s
        A = pruned_weight(r, c, 0.10, 1004 if seed is None else seed)
        return dict(name="pruned 90%% %dx%d fp32 storage (tf32 variant)" % (r, c), A=A, N=(256,), b_seed=2004)
    if index == 4:
        r, c = 4096 // s, 14336 // s
        A = block_sparse(r, c, 16, 0.5, 1005 if seed is None else seed)
        return dict(name="16x16-block 50%% %dx%d fp16" % (r, c), A=A, N=(16, 64, 512), b_seed=2005)
    raise ValueError("configuration index must be 0..4")


def algorithmic_bytes(btcf, N):
    """Compulsory bytes of one SpMM: every array touched once - the tiles, the
    column ids, rowOffset, rowIdx, each B row that is referenced at least once,
    and all of C."""
    s = 4 if btcf["dtype"] == TF32 else 2
    cw = btcf["cw"]
    T, W, M = int(btcf["total_tiles"]), int(btcf["eff_row_windows"]), int(btcf["rows"])
    ids = btcf["tcA2B"]
    U = int(np.unique(ids[ids != 0xFFFFFFFF]).size) if ids.size else 0
    return s * 8 * cw * T + 4 * cw * T + 4 * (W + 1) + 4 * W + s * N * U + s * N * M


def gather_bytes(btcf, N):
    """Same with every gathered B row counted every time it is read."""
    s = 4 if btcf["dtype"] == TF32 else 2
    cw = btcf["cw"]
    T, W, M = int(btcf["total_tiles"]), int(btcf["eff_row_windows"]), int(btcf["rows"])
    ids = btcf["tcA2B"]
    P = int(np.count_nonzero(ids != 0xFFFFFFFF))
    return s * 8 * cw * T + 4 * cw * T + 4 * (W + 1) + 4 * W + s * N * P + s * N * M
