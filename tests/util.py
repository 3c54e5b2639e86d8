"""Helpers shared by the tests."""
import numpy as np

IDX_MAX = 0xFFFFFFFF


def dtype_name(dtype):
    return {0: "fp16", 1: "tf32", 2: "bf16"}[dtype]


def encode(x, dtype):
    """float values -> storage of dtype: uint16 bits (fp16 = 0, bf16 = 2) or float32 (1).
    bf16 goes through torch's CPU conversion, which is independent of both the
    library's and the oracle's."""
    x = np.ascontiguousarray(x, np.float32)
    if dtype == 0:
        return x.astype(np.float16).view(np.uint16)
    if dtype == 2:
        import torch
        return torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    return x


def decode(v, dtype):
    """storage of dtype -> float64."""
    if dtype == 0:
        return np.ascontiguousarray(v).view(np.float16).astype(np.float64)
    if dtype == 2:
        return (np.ascontiguousarray(v).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return np.asarray(v).astype(np.float64)


def random_csr(rng, rows, cols, density, dtype, empty_row_prob=0.0, heavy_rows=()):
    """Duplicate-free random CSR; values are fp16 / bf16 bit patterns or float32."""
    row_lists = []
    for r in range(rows):
        if r in heavy_rows:
            k = max(1, int(cols * 0.8))
        elif rng.random() < empty_row_prob:
            k = 0
        else:
            k = rng.binomial(cols, density)
        c = np.sort(rng.choice(cols, size=min(k, cols), replace=False)).astype(np.uint32)
        row_lists.append(c)
    row_ptr = np.zeros(rows + 1, np.uint32)
    row_ptr[1:] = np.cumsum([len(c) for c in row_lists])
    col_idx = np.concatenate(row_lists).astype(np.uint32) if rows else np.zeros(0, np.uint32)
    v = rng.uniform(-1, 1, col_idx.size).astype(np.float32)
    vals = encode(v, dtype)
    return dict(rows=rows, cols=cols, nnzs=int(col_idx.size), dtype=dtype, row_ptr=row_ptr,
                col_idx=col_idx, values=vals)


def csr_to_dense64(A):
    """Dense float64 copy of a CSR dict."""
    vals = decode(A["values"], A["dtype"])
    D = np.zeros((A["rows"], A["cols"]), np.float64)
    rp = A["row_ptr"]
    for r in range(A["rows"]):
        D[r, A["col_idx"][rp[r]:rp[r + 1]]] = vals[rp[r]:rp[r + 1]]
    return D


def btcf_to_csr(b):
    """Expand tiles through tcA2B / rowIdx back to (row, col, value) triples sorted
    by (row, col): the round trip of the condensed format."""
    cw = b["cw"]
    out = []
    data = b["data"].reshape(-1, 8, cw)
    a2b = b["tcA2B"].reshape(-1, cw)
    for w in range(b["eff_row_windows"]):
        for t in range(b["rowOffset"][w], b["rowOffset"][w + 1]):
            for k in range(cw):
                c = a2b[t, k]
                if c == IDX_MAX:
                    continue
                for r in range(8):
                    v = data[t, r, k]
                    if v != 0:
                        out.append((int(b["rowIdx"][w]) + r, int(c), v))
    out.sort(key=lambda x: (x[0], x[1]))
    return out


def csr_triples(A):
    rp = A["row_ptr"]
    out = []
    for r in range(A["rows"]):
        for i in range(rp[r], rp[r + 1]):
            out.append((r, int(A["col_idx"][i]), A["values"][i]))
    return out


def half_ulp_distance(a_bits, b_bits):
    """Distance in units of the last place between two arrays of 16-bit float bit
    patterns (fp16 or bf16: sign-magnitude ordering holds for both)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def built_depth(hs, stages):
    """The prefetch depth a test asks for, or the default-build depth 3 in its place when the library holds
    depths 2, 3 and 4 only (1, 6 and 8 are built with EXPERIMENTAL=1)."""
    return stages if stages in (0, 2, 3, 4) or hs.has_experimental() else 3
