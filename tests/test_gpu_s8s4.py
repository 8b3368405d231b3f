"""s8 x s4 -> s32 on the matrix cores (the thin kernel's 4-bit path) against the
oracle's restatement of mmt4d_tile_generic.c:11-51, bit for bit, on full-range
inputs: every s8 value on the LHS and every byte value (both nibbles from -8 to
7) on the RHS, so that the nibble order, the sign extension and the even/odd
pairing of LHS bytes are all exercised."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

TF = uk.MMT4D_TYPE_S8S4S32


def _full_range(c, rng):
    lhs = rng.integers(-128, 128, c.M * c.lhs_stride0 + c.lhs_offset + 64, dtype=np.int8).view(np.uint8)
    rhs = rng.integers(0, 256, (c.N * c.rhs_stride0 + c.rhs_offset) // 2 + 64, dtype=np.uint8)
    out = rng.integers(-2 ** 31, 2 ** 31, c.M * c.out_stride0 + c.out_offset + 16,
                       dtype=np.int64).astype(np.int32).view(np.uint8)
    return lhs, rhs, out


@pytest.mark.gpu
@pytest.mark.parametrize("M0,N0,K0", [(16, 16, 16), (32, 16, 16), (8, 8, 32), (16, 32, 64),
                                      (1, 16, 16), (24, 20, 32)])
def test_s8s4_thin_kernel_full_range(gpu, oracle, M0, N0, K0):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    step = 64 // K0                      # K tiles per 64-element step
    shapes = [(1, 1, step), (1, 7, 5 * step), (2, 3, 16 * step), (3, 40, 9 * step),
              (max(1, 100 // M0), 5, 4 * step), (1, 33, 37 * step)]
    for si, (M1, N1, K1) in enumerate(shapes):
        for ci, c in enumerate(T.mmt4d_cases(TF, M0, N0, K0, seed=500 + si, slack=16,
                                             shapes=((M1, N1, K1),))):
            rng = np.random.default_rng(10 * si + ci)
            lhs, rhs, out0 = _full_range(c, rng)
            want = out0.copy()
            G.run_mmt4d_case(oracle, c, lhs, rhs, want)
            got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
            assert lib.last_kernel_name() == "mmt4d_mfma_thin_s8s4", (c.label(), lib.last_kernel_name())
            assert np.array_equal(got, want), c.label()
    # K not in whole steps, or a tile depth the kernel does not take: generic, same answer
    for (M1, N1, K1, k0) in ((2, 3, step + 1 if step > 1 else 0, K0), (2, 3, 8, 8)):
        if K1 == 0:
            continue
        c = T.Mmt4dCase(TF, M1, N1, K1, M0, N0, k0, K1 * M0 * k0, K1 * N0 * k0, N1 * M0 * N0, 0, 0, 0)
        rng = np.random.default_rng(77)
        lhs, rhs, out0 = _full_range(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == "mmt4d_generic"
        assert np.array_equal(got, want), c.label()


@pytest.mark.gpu
def test_s8s4_decode_shape_equals_integer_product(gpu):
    """A decode-sized call (16 rows, K = 4096, N = 4096, tiles 16x16x32 with
    ACCUMULATE) against the exact integer product of the unpacked operands."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M0, N0, K0 = 16, 16, 32
    M1, N1, K1 = 1, 256, 128
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    lhs = torch.randint(-128, 128, (M1, K1, M0, K0), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(0, 256, (N1, K1, N0, K0 // 2), generator=g, device="cuda", dtype=torch.uint8)
    out = torch.randint(-10 ** 6, 10 ** 6, (M1, N1, M0, N0), generator=g, device="cuda", dtype=torch.int32)
    init = out.clone()
    lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, TF | uk.MMT4D_ACCUMULATE | 0x200)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_mfma_thin_s8s4"
    r = rhs.cpu().to(torch.int64)
    lo, hi = r & 0xF, r >> 4
    lo = torch.where(lo >= 8, lo - 16, lo)
    hi = torch.where(hi >= 8, hi - 16, hi)
    vals = torch.stack([lo, hi], dim=-1).reshape(N1, K1, N0, K0)        # element 2h = low nibble
    a = lhs.cpu().to(torch.int64).permute(0, 2, 1, 3).reshape(M1 * M0, K1 * K0)
    b = vals.permute(0, 2, 1, 3).reshape(N1 * N0, K1 * K0)
    want = (a @ b.T).reshape(M1, M0, N1, N0).permute(0, 2, 1, 3) + init.cpu().to(torch.int64)
    assert torch.equal(out.cpu().to(torch.int64), want)


@pytest.mark.gpu
@pytest.mark.parametrize("M0,N0,K0", [(16, 16, 16), (16, 16, 32), (32, 8, 64), (24, 20, 32), (1, 16, 16),
                                      (8, 8, 8), (16, 16, 2), (4, 8, 4)])
def test_s8s4_many_rows_run_on_expanded_weights(gpu, oracle, M0, N0, K0):
    """From 512 rows on the 4-bit weights are expanded to s8 once and the s8
    kernels run on the copy: full-range inputs, ACCUMULATE off and on, loose
    strides and offsets (the reference's case grid), bit for bit against the
    oracle; 511 rows still run on the thin kernel, or, for tile rows under 16
    elements (arm64's 8x8x8 among them: arch/arm_64/mmt4d_arm_64_dotprod.c:85),
    on the scalar one."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    step = max(1, 64 // K0)
    rows = -(-512 // M0)
    shapes = [(rows, 3, 2 * step), (rows + 3, 9, 5 * step), (2 * rows + 1, 1, step)]
    for si, (M1, N1, K1) in enumerate(shapes):
        for ci, c in enumerate(T.mmt4d_cases(TF, M0, N0, K0, seed=900 + si, slack=16,
                                             shapes=((M1, N1, K1),))):
            rng = np.random.default_rng(100 * si + ci)
            lhs, rhs, out0 = _full_range(c, rng)
            want = out0.copy()
            G.run_mmt4d_case(oracle, c, lhs, rhs, want)
            got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
            assert lib.last_kernel_name() == "mmt4d_mfma_s8s4_expanded", (c.label(), lib.last_kernel_name())
            assert np.array_equal(got, want), c.label()
    if (511 // M0) * M0 >= 64:
        c = next(iter(T.mmt4d_cases(TF, M0, N0, K0, seed=7, slack=16, shapes=((511 // M0, 3, 2 * step),))))
        lhs, rhs, out0 = _full_range(c, np.random.default_rng(3))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == ("mmt4d_mfma_thin_s8s4" if K0 >= 16 else "mmt4d_generic"), \
            lib.last_kernel_name()
        assert np.array_equal(got, want), c.label()


@pytest.mark.gpu
def test_s8s4_prefill_shape_equals_integer_product(gpu):
    """A prefill-sized call (2048 rows against 4096 x 2048 4-bit weights, tiles
    16x16x32, ACCUMULATE) against the exact integer product of the unpacked
    operands, twice in a row with different weights (the second call reuses the
    library's buffer for the expanded weights), and once through the entry
    point that may not allocate, which keeps the thin kernel."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M0, N0, K0 = 16, 16, 32
    M1, N1, K1 = 128, 256, 64
    g = torch.Generator(device="cuda"); g.manual_seed(11)
    for rep in range(3):
        lhs = torch.randint(-128, 128, (M1, K1, M0, K0), generator=g, device="cuda", dtype=torch.int8)
        rhs = torch.randint(0, 256, (N1, K1, N0, K0 // 2), generator=g, device="cuda", dtype=torch.uint8)
        out = torch.randint(-10 ** 6, 10 ** 6, (M1, N1, M0, N0), generator=g, device="cuda", dtype=torch.int32)
        init = out.clone()
        call = lib.mmt4d_no_alloc if rep == 2 else lib.mmt4d
        call(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
             N1 * M0 * N0, M1, N1, K1, M0, N0, K0, TF | uk.MMT4D_ACCUMULATE | 0x200)
        lib.synchronize()
        assert lib.last_kernel_name() == ("mmt4d_mfma_thin_s8s4" if rep == 2 else "mmt4d_mfma_s8s4_expanded")
        r = rhs.to(torch.int64)
        lo, hi = r & 0xF, r >> 4
        lo = torch.where(lo >= 8, lo - 16, lo)
        hi = torch.where(hi >= 8, hi - 16, hi)
        vals = torch.stack([lo, hi], dim=-1).reshape(N1, K1, N0, K0)        # element 2h = low nibble
        a = lhs.permute(0, 2, 1, 3).reshape(M1 * M0, K1 * K0).double()
        b = vals.permute(0, 2, 1, 3).reshape(N1 * N0, K1 * K0).double()
        # (every partial sum is an integer below 2^53: the f64 product is exact)
        want = (a @ b.T).to(torch.int64).reshape(M1, M0, N1, N0).permute(0, 2, 1, 3) + init.to(torch.int64)
        assert torch.equal(out.to(torch.int64), want), rep


@pytest.mark.gpu
def test_prepared_operand_buffer_is_reported_and_can_be_released(gpu):
    """The buffer for the expanded weights is kept for the next call on the same
    stream, shows in iree_uk_amd_workspace_bytes, is freed by
    iree_uk_amd_release_workspaces, and a later call allocates it again."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M0, N0, K0, M1, N1, K1 = 16, 16, 16, 32, 16, 8
    lhs = torch.randint(-128, 128, (M1 * K1 * M0 * K0,), device="cuda", dtype=torch.int8)
    rhs = torch.randint(0, 256, (N1 * K1 * N0 * K0 // 2,), device="cuda", dtype=torch.uint8)
    out = torch.zeros(M1 * N1 * M0 * N0, device="cuda", dtype=torch.int32)

    def call():
        lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
                  N1 * M0 * N0, M1, N1, K1, M0, N0, K0, TF | 0x200)
        lib.synchronize()
        assert lib.last_kernel_name() == "mmt4d_mfma_s8s4_expanded"
        return out.clone()

    lib.release_workspaces()
    assert lib.workspace_bytes() == 0
    first = call()
    held = lib.workspace_bytes()
    assert held >= N1 * K1 * N0 * K0
    allocs = lib.device_alloc_count()
    second = call()
    assert lib.device_alloc_count() == allocs and lib.workspace_bytes() == held   # reused, not grown
    assert lib.release_workspaces() == 0 and lib.workspace_bytes() == 0
    third = call()
    assert lib.workspace_bytes() == held
    assert torch.equal(first, second) and torch.equal(first, third)
