"""iree_uk_amd_mmt4d_no_alloc, the mmt4d entry point that allocates nothing
(its K-split workspace is a static device array of the library), against
iree_uk_mmt4d on the same inputs, through the C-ABI: bit for bit, floats
included (both take the same kernel with the same split of K). Two calls in a
row share the array, the second on a smaller problem; a call whose split needs
more than the array holds and a call on host operands are refused with their
own status and write nothing."""
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


def test_no_alloc_refuses_what_it_cannot_serve(gpu):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    # 64 rows against 6400 columns with 8 K slices: 200 blocks x 8 slices x 8 KiB
    # of partials is more than the static array's 8 MiB.
    assert lib.no_alloc_scratch_bytes() == (8 << 20) + 16384 * 4
    lhs, rhs, out0, args = _problem(torch, uk.MMT4D_TYPE_S8S8S32, 64, 6400, 8192, 16, 16, 16, 60, False)
    lib.set_k_slices(8)
    try:
        got = out0.clone()
        lib.mmt4d_no_alloc(*args(got), check=False)
        assert lib.last_status() == uk.STATUS_SCRATCH_TOO_SMALL
        assert "scratch" in lib.last_status_string()
        lib.synchronize()
        assert torch.equal(got, out0), "a refused call writes nothing"
        want = out0.clone()
        lib.mmt4d(*args(want))          # the allocating entry point serves it
        lib.synchronize()
        assert lib.last_k_slices() == 8
    finally:
        lib.set_k_slices(0)
    # host operands would need staging through a device allocation
    a = np.zeros(16 * 16, np.int8)
    o = np.zeros(16 * 16, np.int32)
    lib.mmt4d_no_alloc(a.ctypes.data, 0, 256, a.ctypes.data, 0, 256, o.ctypes.data, 0, 256, 1, 1, 1,
                       16, 16, 16, uk.MMT4D_TYPE_S8S8S32, check=False)
    assert lib.last_status() == uk.STATUS_NEEDS_ALLOCATION
    assert not o.any()
