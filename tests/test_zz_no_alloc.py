"""hspmm_run_static - the entry point that allocates nothing: the partial sums of cut windows go to a
fixed array of device memory that the library holds, not to a buffer of the plan.  Its output must be
bit-identical to hspmm_run's, call after call, also when a later call is smaller than the one before
(the array keeps the earlier call's contents).  Needs a real MI355X: run with -m gpu."""
import numpy as np
import pytest

from util import random_csr
from test_spmm_gpu import torch_cuda, convert, make_b, oracle_spmm, assert_parity  # noqa: F401

pytestmark = pytest.mark.gpu


def _device_buffers(torch, B, rows, N, dtype):
    if dtype != 1:
        dB = torch.from_numpy(np.ascontiguousarray(B, np.uint16).view(np.int16)).cuda()
        dC = torch.empty((rows, N), dtype=torch.int16, device="cuda")
    else:
        dB = torch.from_numpy(np.ascontiguousarray(B, np.float32)).cuda()
        dC = torch.empty((rows, N), dtype=torch.float32, device="cuda")
    return dB, dC


def _poison(dC, dtype):
    dC.fill_(0x7E01 if dtype != 1 else float("nan"))


def _result(dC, dtype):
    out = dC.cpu().numpy()
    return out.view(np.uint16) if dtype != 1 else out


def _cases(hs, rng, dtype):
    """(name, CSR, N, configure keywords): first a large call, then a smaller one; both with windows cut
    across waves (gather kernels, two kernels per call), then the LDS-staging kernels with chunk sums."""
    heavy = dict(producer_warp_group_num=16)
    yield "gather, large", random_csr(rng, 640, 6000, 0.004, dtype, 0.1, (5, 17, 300)), 128, heavy
    yield "gather, small", random_csr(rng, 200, 3000, 0.004, dtype, 0.1, (9,)), 64, heavy
    yield "panel, large", random_csr(rng, 480, 4000, 0.1, dtype, 0.05), 256, {}
    yield "panel, small", random_csr(rng, 160, 2000, 0.1, dtype, 0.05), 128, {}


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_static_scratch_entry_point_matches_hspmm_run(torch_cuda, hs, oracle, dtype):
    torch = torch_cuda
    rng = np.random.default_rng(700 + dtype)
    stream = torch.cuda.current_stream().cuda_stream
    for name, A, N, knobs in _cases(hs, rng, dtype):
        b = convert(hs, A)
        hs.configure(**knobs)
        try:
            plan = hs.Plan(b)
        finally:
            hs.configure()
        info = plan.info()
        B = make_b(rng, A["cols"], N, dtype)
        dB, dC = _device_buffers(torch, B, A["rows"], N, dtype)
        # 16-bit types, one wave covers all of N: the launch wants the partition whose workgroups add their
        # waves' sums, which hspmm_create has not built - the entry point must refuse instead of building it
        if info["n_panels"] == 0 and dtype != 1:
            with pytest.raises(hs.HspmmError) as e:
                plan.run_static(dB.data_ptr(), dC.data_ptr(), N, stream)
            assert "hspmm_prepare" in str(e.value)
        plan.prepare(N)
        _poison(dC, dtype)
        torch.cuda.synchronize()
        # the device allocator itself: free memory of the device before and after the call (the plan's own
        # accounting, which also counts arrival counters and superseded buffers, must agree)
        before = torch.cuda.mem_get_info()[0], plan.info()["device_bytes"]
        plan.run_static(dB.data_ptr(), dC.data_ptr(), N, stream)
        torch.cuda.synchronize()
        after = torch.cuda.mem_get_info()[0], plan.info()["device_bytes"]
        got = _result(dC, dtype)
        assert after[1] == before[1], name + ": the plan's device memory changed"
        assert after[0] >= before[0], name + ": %d bytes of device memory were allocated by the call" % (before[0] - after[0])
        # the existing entry point, same plan, same inputs
        _poison(dC, dtype)
        plan.run(dB.data_ptr(), dC.data_ptr(), N, stream)
        torch.cuda.synchronize()
        want = _result(dC, dtype)
        family = plan.info()["last_kernel_family"]
        assert family == (3 if name.startswith("panel") else 2), (name, family)
        if name.startswith("gather"):
            assert info["n_split_windows"] > 0, name + ": no window is cut, nothing would use scratch memory"
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), name + ": differs from hspmm_run"
        ref, mag = oracle_spmm(oracle, A, B, N)
        assert_parity(got, ref, mag, dtype, name)
        # again, into the array the call above left its sums in
        _poison(dC, dtype)
        plan.run_static(dB.data_ptr(), dC.data_ptr(), N, stream)
        torch.cuda.synchronize()
        assert np.array_equal(_result(dC, dtype).view(np.uint8), want.view(np.uint8)), name + ": second call differs"
        plan.close()


def test_static_scratch_entry_point_with_a_single_feature(torch_cuda, hs, oracle):
    """Matrix times vector in a 16-bit type goes through a buffer of the plan's (B and C widened to words): the
    entry point refuses until hspmm_prepare(plan, 1) has made it, then gives the bits of hspmm_run."""
    torch = torch_cuda
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(78)
    A = random_csr(rng, 300, 3000, 0.004, 0, 0.2, (5, 100, 299))
    b = convert(hs, A)
    hs.configure(producer_warp_group_num=16)                        # (cut windows: partial sums in the fixed array)
    try:
        plan = hs.Plan(b)
    finally:
        hs.configure()
    B = make_b(rng, A["cols"], 1, 0)
    dB, dC = _device_buffers(torch, B, A["rows"], 1, 0)
    with pytest.raises(hs.HspmmError) as e:
        plan.run_static(dB.data_ptr(), dC.data_ptr(), 1, stream)
    assert "hspmm_prepare" in str(e.value)
    plan.prepare(1)
    before = plan.info()["device_bytes"]
    for _ in range(2):
        _poison(dC, 0)
        plan.run_static(dB.data_ptr(), dC.data_ptr(), 1, stream)
        torch.cuda.synchronize()
        got = _result(dC, 0)
        assert plan.info()["last_kernel_family"] == 2 and plan.info()["device_bytes"] == before
    _poison(dC, 0)
    plan.run(dB.data_ptr(), dC.data_ptr(), 1, stream)
    torch.cuda.synchronize()
    assert np.array_equal(got.view(np.uint8), _result(dC, 0).view(np.uint8))
    ref, mag = oracle_spmm(oracle, A, B, 1)
    assert_parity(got, ref, mag, 0, "single feature")
    plan.close()


def test_static_scratch_entry_point_rejects_what_does_not_fit(torch_cuda, hs):
    """A launch whose partial sums exceed the fixed array is refused with a message that says so."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    # every window far longer than a range, many ranges, wide N: tens of MB of partial sums
    A = random_csr(rng, 2048, 8192, 0.25, 0)
    b = convert(hs, A)
    hs.set_kernel_mode(3)
    hs.configure(producer_warp_group_num=16)
    try:
        plan = hs.Plan(b)
    finally:
        hs.configure()
        hs.set_kernel_mode(0)
    N = 2048
    plan.prepare(N)
    assert plan.info()["device_bytes"] > 2 * (32 << 20)          # the plan's own buffer for this N is far larger
    dB = torch.zeros((8192, N), dtype=torch.int16, device="cuda")
    dC = torch.zeros((2048, N), dtype=torch.int16, device="cuda")
    with pytest.raises(hs.HspmmError) as e:
        plan.run_static(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)
    assert "fixed array holds" in str(e.value), str(e.value)
    plan.run(dB.data_ptr(), dC.data_ptr(), N, torch.cuda.current_stream().cuda_stream)   # the allocating entry point serves it
    torch.cuda.synchronize()
    assert not dC.any().item()
    plan.close()


def test_prepare_covers_rows_that_start_on_odd_halves(torch_cuda, hs, oracle):
    """hspmm_prepare builds for every alignment of B and C, also a 16-bit B or C that starts on an odd half: that
    launch takes one-word loads in blocks of 32 features, i.e. several feature blocks, another partition and another
    amount of partial sums than the aligned launches.  hspmm_run_static, which builds nothing, must then run it."""
    torch = torch_cuda
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(79)
    A = random_csr(rng, 64, 6000, 0.3, 0, 0.0, (3, 40))            # every unit far longer than a range
    b = convert(hs, A)
    hs.set_kernel_mode(3)                                           # (gather kernels, whatever the density)
    try:
        plan = hs.Plan(b)
    finally:
        hs.set_kernel_mode(0)
    N = 256
    B = make_b(rng, A["cols"], N, 0)
    flatB = torch.zeros(A["cols"] * N + 1, dtype=torch.int16, device="cuda")
    flatC = torch.zeros(A["rows"] * N + 1, dtype=torch.int16, device="cuda")
    flatB[1:] = torch.from_numpy(np.ascontiguousarray(B, np.uint16).view(np.int16).ravel()).cuda()
    pB, pC = flatB.data_ptr() + 2, flatC.data_ptr() + 2             # one half into their allocations
    plan.prepare(N)
    torch.cuda.synchronize()
    before = torch.cuda.mem_get_info()[0], plan.info()["device_bytes"]
    plan.run_static(pB, pC, N, stream)
    torch.cuda.synchronize()
    assert plan.info()["device_bytes"] == before[1] and torch.cuda.mem_get_info()[0] >= before[0]
    got = flatC[1:].cpu().numpy().view(np.uint16).reshape(A["rows"], N)
    ref, mag = oracle_spmm(oracle, A, B, N)
    assert_parity(got, ref, mag, 0, "B and C on odd halves")
    assert int(flatC[0].item()) == 0                                # nothing in front of C was written
    plan.close()


def test_first_launch_after_prepare_takes_the_prepared_buffers(torch_cuda, hs, oracle):
    """hspmm_prepare on a plan that has not launched yet makes one set of buffers; the first stream that launches
    the plan - here a stream of its own, not the default one - takes that set instead of allocating another."""
    torch = torch_cuda
    rng = np.random.default_rng(80)
    A = random_csr(rng, 300, 3000, 0.004, 0, 0.2, (5, 100, 299))
    b = convert(hs, A)
    hs.configure(producer_warp_group_num=16)                        # (cut windows: partial sums and counters)
    try:
        plan = hs.Plan(b)
    finally:
        hs.configure()
    N = 128
    B = make_b(rng, A["cols"], N, 0)
    dB, dC = _device_buffers(torch, B, A["rows"], N, 0)
    plan.prepare(N)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        dC.zero_()                      # (the runtime's own memory for a new stream's first launch exists after this)
    torch.cuda.synchronize()
    before = torch.cuda.mem_get_info()[0], plan.info()["device_bytes"]
    plan.run(dB.data_ptr(), dC.data_ptr(), N, side.cuda_stream)
    side.synchronize()
    assert plan.info()["device_bytes"] == before[1], "the first launch allocated buffers of its own"
    assert torch.cuda.mem_get_info()[0] >= before[0]
    ref, mag = oracle_spmm(oracle, A, B, N)
    assert_parity(_result(dC, 0), ref, mag, 0, "first launch after prepare")
    plan.close()
