"""iree_uk_amd_mmt4d_no_alloc, the mmt4d entry point that allocates nothing
(its K-split workspace is a static device array of the library), through the
C-ABI: against the exact integer product and against iree_uk_mmt4d on the same
inputs, bit for bit, floats included (both take the same kernel with the same
split of K). Two calls in a row share the array, the second on a smaller
problem; a call whose split would need more than the array holds runs without
the split; a call on host operands is refused with its own status and writes
nothing; the call replays from a captured HIP graph."""
import threading

import numpy as np
import pytest

from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu


def _problem(torch, tf, Mrows, N, K, M0, N0, K0, seed, accumulate):
    g = torch.Generator(device="cuda"); g.manual_seed(seed)
    M1, N1, K1 = -(-Mrows // M0), N // N0, K // K0
    if tf == uk.MMT4D_TYPE_S8S8S32:
        lhs = torch.randint(-128, 128, (M1 * K1 * M0 * K0,), generator=g, device="cuda", dtype=torch.int8)
        rhs = torch.randint(-128, 128, (N1 * K1 * N0 * K0,), generator=g, device="cuda", dtype=torch.int8)
        out = torch.randint(-2 ** 15, 2 ** 15, (M1 * N1 * M0 * N0,), generator=g, device="cuda",
                            dtype=torch.int32)
    else:
        lhs = torch.randn(M1 * K1 * M0 * K0, generator=g, device="cuda").to(torch.float16)
        rhs = torch.randn(N1 * K1 * N0 * K0, generator=g, device="cuda").to(torch.float16)
        out = torch.randn(M1 * N1 * M0 * N0, generator=g, device="cuda")
    flags = tf | (uk.MMT4D_ACCUMULATE if accumulate else 0)
    args = lambda o: (lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, o.data_ptr(), 0,
                      N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags)
    return lhs, rhs, out, args


def _integer_product(torch, lhs, rhs, out0, Mrows, N, K, M0, N0, K0, accumulate):
    """The tiled s32 result from the s8 operands by 64-bit integer arithmetic on
    the host (a closed form, independent of every kernel)."""
    M1, N1, K1 = -(-Mrows // M0), N // N0, K // K0
    a = lhs.view(M1, K1, M0, K0).permute(0, 2, 1, 3).reshape(M1 * M0, K).cpu().to(torch.int64)
    b = rhs.view(N1, K1, N0, K0).permute(0, 2, 1, 3).reshape(N, K).cpu().to(torch.int64)
    c = a @ b.T
    if accumulate:
        c = c + out0.view(M1, N1, M0, N0).permute(0, 2, 1, 3).reshape(M1 * M0, N).cpu().to(torch.int64)
    return c.to(torch.int32).view(M1, M0, N1, N0).permute(0, 2, 1, 3).reshape(-1)


def test_no_alloc_first_call_of_a_fresh_thread_allocates_nothing_and_is_exact(gpu):
    """The very first mmt4d call of a new host thread, on a stream of its own,
    through the entry point that allocates nothing: the K split engages (so the
    static array is what it used: this thread owns no workspace), free device
    memory is what it was before the call, and the integers are exact. The same
    call then replays from a captured graph."""
    lib, torch = gpu
    Mrows, N, K, M0, N0, K0 = 16, 1024, 14336, 16, 16, 16
    lhs, rhs, out0, args = _problem(torch, uk.MMT4D_TYPE_S8S8S32, Mrows, N, K, M0, N0, K0, 70, True)
    want = _integer_product(torch, lhs, rhs, out0, Mrows, N, K, M0, N0, K0, True)
    got, replayed = out0.clone(), out0.clone()
    # The runtime loads the library's code objects, the one that holds the
    # static array among them, when they are first used: one call through this
    # same entry point on the test's own thread makes them resident. It owns
    # no workspace either (this entry point never creates one), so nothing of
    # it can serve the fresh thread below.
    warm_in = torch.zeros(256, device="cuda", dtype=torch.int8)
    w_lhs, w_rhs, w_out, w_args = _problem(torch, uk.MMT4D_TYPE_S8S8S32, 16, 512, 4096, 16, 16, 16, 71, False)
    lib.set_k_slices(0)
    lib.mmt4d_no_alloc(*w_args(w_out))
    lib.synchronize()
    assert lib.last_k_slices() > 1
    torch.cuda.synchronize()
    result = {}

    def worker():
        try:
            stream = torch.cuda.Stream()
            lib.set_pointer_mode(uk.POINTER_MODE_DEVICE)
            lib.set_stream(stream.cuda_stream)
            lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
            lib.set_k_slices(0)
            # The runtime sets up a new stream's queue at its first launch (and
            # takes device memory for it): let that launch be someone else's.
            with torch.cuda.stream(stream):
                warm_in.zero_()
            stream.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            allocs_before = lib.device_alloc_count()
            lib.mmt4d_no_alloc(*args(got))
            lib.synchronize()
            result["allocs"] = lib.device_alloc_count() - allocs_before
            result["free_delta"] = free_before - torch.cuda.mem_get_info()[0]
            result["slices"] = lib.last_k_slices()
            result["kernel"] = lib.last_kernel_name()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                lib.mmt4d_no_alloc(*args(replayed))
            torch.cuda.synchronize()
            reps = []
            for _ in range(2):
                replayed.copy_(out0)          # eager work between the replays
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                reps.append(replayed.cpu().clone())
            result["replays"] = reps
            # The ordinary entry point on the same problem and thread does allocate
            # (its K-split workspace, once): the counter sees that.
            allocs_before = lib.device_alloc_count()
            lib.mmt4d(*args(replayed))
            lib.synchronize()
            result["allocs_ordinary"] = lib.device_alloc_count() - allocs_before
            lib.set_stream(None)
            lib.set_pointer_mode(uk.POINTER_MODE_AUTO)
        except BaseException as e:  # noqa: BLE001 - reported by the test thread
            result["error"] = e

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert "error" not in result, result.get("error")
    assert result["slices"] > 1, (result["slices"], result["kernel"])
    # The library's own count of its hipMalloc calls is the evidence; the
    # device's free memory backs it up, up to what the HIP runtime may take for
    # itself at any moment (it moves in chunks of 64 MiB).
    assert result["allocs"] == 0, result["allocs"]
    assert result["allocs_ordinary"] == 1, result["allocs_ordinary"]
    assert result["free_delta"] < (64 << 20), result["free_delta"]
    assert torch.equal(got.cpu(), want)
    for rep in result["replays"]:
        assert torch.equal(rep, want)


@pytest.mark.parametrize("tf", [uk.MMT4D_TYPE_S8S8S32, uk.MMT4D_TYPE_F16F16F32])
def test_no_alloc_equals_mmt4d_on_two_calls_in_a_row(gpu, tf):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_k_slices(0)
    # A decode step against a matrix of few rows and a long K (the K split
    # engages), then a smaller one of the same kind, then one the split does
    # not touch at all (a square problem).
    shapes = [(16, 1024, 14336, 16, 16, 16, True), (16, 512, 4096, 16, 16, 16, False),
              (256, 512, 1024, 16, 16, 16, True)]
    for i, (Mrows, N, K, M0, N0, K0, acc) in enumerate(shapes):
        lhs, rhs, out0, args = _problem(torch, tf, Mrows, N, K, M0, N0, K0, 50 + i, acc)
        want = out0.clone()
        lib.mmt4d(*args(want))
        lib.synchronize()
        slices_ref, kernel_ref = lib.last_k_slices(), lib.last_kernel_name()
        got = out0.clone()
        lib.mmt4d_no_alloc(*args(got))
        lib.synchronize()
        assert lib.last_kernel_name() == kernel_ref
        assert lib.last_k_slices() == slices_ref
        if i < 2:
            assert slices_ref > 1, "the decode-shaped cases are meant to split K"
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (i, kernel_ref)
        assert not torch.equal(got.view(torch.int32), out0.view(torch.int32))
        if tf == uk.MMT4D_TYPE_S8S8S32:
            exact = _integer_product(torch, lhs, rhs, out0, Mrows, N, K, M0, N0, K0, acc)
            assert torch.equal(got.cpu(), exact), i


def test_no_alloc_runs_unsplit_what_the_array_cannot_hold_and_refuses_host_operands(gpu):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    # 64 rows against 6400 columns with 8 K slices: 200 blocks x 8 slices x 8 KiB
    # of partials is more than the static array's 8 MiB.
    assert lib.no_alloc_scratch_bytes() == (8 << 20) + 16384 * 4
    Mrows, N, K, M0, N0, K0 = 64, 6400, 8192, 16, 16, 16
    lhs, rhs, out0, args = _problem(torch, uk.MMT4D_TYPE_S8S8S32, Mrows, N, K, M0, N0, K0, 60, False)
    lib.set_k_slices(8)
    try:
        got = out0.clone()
        lib.mmt4d_no_alloc(*args(got))
        lib.synchronize()
        assert lib.last_k_slices() == 1, "a split that does not fit the array is not made"
        assert lib.last_kernel_name().startswith("mmt4d_mfma_thin"), lib.last_kernel_name()
        assert torch.equal(got.cpu(), _integer_product(torch, lhs, rhs, out0, Mrows, N, K, M0, N0, K0, False))
        want = out0.clone()
        lib.mmt4d(*args(want))          # the allocating entry point makes the split
        lib.synchronize()
        assert lib.last_k_slices() == 8
        assert torch.equal(got, want)
    finally:
        lib.set_k_slices(0)
    # host operands would need staging through a device allocation
    a = np.zeros(16 * 16, np.int8)
    o = np.zeros(16 * 16, np.int32)
    lib.mmt4d_no_alloc(a.ctypes.data, 0, 256, a.ctypes.data, 0, 256, o.ctypes.data, 0, 256, 1, 1, 1,
                       16, 16, 16, uk.MMT4D_TYPE_S8S8S32, check=False)
    assert lib.last_status() == uk.STATUS_NEEDS_ALLOCATION
    assert not o.any()
