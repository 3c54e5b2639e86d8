"""The synthetic inputs of the benchmark configurations are functions of their seeds alone: raw words of the
counter-based Philox generator, turned into uniforms, bounded integers and normals by the transforms of
hopper_spmm_amd.generators.Stream (no distribution method of numpy's, which may change between versions)."""
import hashlib

import numpy as np
import pytest

import hopper_spmm_amd.generators as G


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()[:24]


# (configuration, shrink) -> nnz, digest of row_ptr | col_idx | values
PINNED = {
    (0, 4): (10401, "525ac35ce8497f79ecd68dbb"),
    (1, 8): (130948, "bbd86f8dcd4690b3cd3e16af"),
    (2, 32): (467930, "54915bc6e70072f14ff3e36a"),
    (3, 8): (70451, "bc23778e8131a5700c3a56fc"),
    (4, 8): (460544, "b1c81ba0099dc22b8e0c2658"),
}


@pytest.mark.parametrize("index,shrink", sorted(PINNED))
def test_configurations_are_pinned(index, shrink):
    A = G.make_config(index, shrink)["A"]
    nnz, want = PINNED[(index, shrink)]
    assert A["nnzs"] == nnz
    assert digest(A["row_ptr"], A["col_idx"], A["values"]) == want


def test_dense_b_is_pinned():
    assert digest(G.dense_b(257, 48, 2003, G.FP16)) == "d809f7e088bdb089ff281115"
    assert digest(G.dense_b(257, 48, 2003, G.TF32)) == "268e958f5121e32429035a6c"
    assert digest(G.dense_b(31, 3, 7, G.BF16)) == "6eb610663df6b5f35b97a682"


def test_first_words_of_the_stream():
    """The transforms, spelled out on the first raw words of a seed."""
    raw = np.random.Philox(42).random_raw(4)
    s = G.Stream(42)
    u = s.uniform32(3)                                     # low half, high half of word 0, low half of word 1
    assert u[0] == np.float32((int(raw[0]) & 0xFFFFFFFF) >> 8) / np.float32(1 << 24)
    assert u[1] == np.float32(int(raw[0]) >> 40) / np.float32(1 << 24)
    assert u[2] == np.float32((int(raw[1]) & 0xFFFFFFFF) >> 8) / np.float32(1 << 24)
    d = s.uniform64(-1.0, 1.0, 1)                          # word 2 (the unused half of word 1 is dropped)
    assert d[0] == -1.0 + 2.0 * ((int(raw[2]) >> 11) / 2.0 ** 53)
    k = s.below(1 << 10, 1)
    assert k[0] == (int(raw[3]) & 0xFFFFFFFF) >> 22


def test_normals_are_normal_and_do_not_depend_on_the_chunking(monkeypatch):
    x = G.Stream(9).normal32((1000, 333)).astype(np.float64).ravel()
    assert abs(x.mean()) < 5e-3 and abs(x.std() - 1.0) < 5e-3
    assert abs((np.abs(x) > 1.959964).mean() - 0.05) < 2e-3
    assert abs((x ** 3).mean()) < 2e-2 and abs((x ** 4).mean() - 3.0) < 5e-2
    assert abs(np.corrcoef(x[0::2], x[1::2])[0, 1]) < 5e-3          # the two values of a pair
    monkeypatch.setattr(G, "_CHUNK", 1000)
    y = G.Stream(9).normal32((1000, 333)).astype(np.float64).ravel()
    assert np.array_equal(x, y)
    assert G.Stream(9).normal32(7).shape == (7,) and np.array_equal(G.Stream(9).normal32(7), x[:7].astype(np.float32))


def test_bounded_integers_cover_their_range():
    k = G.Stream(3).below(1000, 200000)
    assert k.min() == 0 and k.max() == 999
    assert abs(np.bincount(k, minlength=1000) / 200.0 - 1.0).max() < 0.35
