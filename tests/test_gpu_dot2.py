"""The 16-bit integer LHS types (s16 x s16, s16 x s8, s16 x u4 -> s32) on the
vector dot-product kernel: bit-exact against the oracle, for the reference's
own x86 tile shapes (16x16x2 VNNI, 1x32x8 for u4) and odd
ones, single tiles to several workgroups, loose strides and odd offsets."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

TILES = [(uk.MMT4D_TYPE_S16S16S32, 16, 16, 2), (uk.MMT4D_TYPE_S16S16S32, 7, 3, 4),
         (uk.MMT4D_TYPE_S16S16S32, 8, 8, 64), (uk.MMT4D_TYPE_S16S8S32, 16, 16, 2),
         (uk.MMT4D_TYPE_S16S8S32, 4, 6, 16), (uk.MMT4D_TYPE_S16U4S32, 1, 32, 8),
         (uk.MMT4D_TYPE_S16U4S32, 5, 3, 2), (uk.MMT4D_TYPE_S16U4S32, 16, 16, 32)]


def _shapes(M0, N0, K0):
    """Tile counts: the reference grid's small cases, K below and above one
    32-element step with a remainder, and blocks of 64 x 64 outputs that are
    ragged in both directions."""
    m_blk, n_blk = -(-64 // M0), -(-64 // N0)
    k_step = max(1, 32 // K0)
    return ((1, 1, 1), (2, 3, 5), (1, 1, 3 * k_step + 1), (m_blk + 1, 1, 2),
            (1, 2 * n_blk + 1, k_step), (2 * m_blk + 1, n_blk + 2, 5 * k_step + 1), (0, 2, 2), (2, 2, 0))


@pytest.mark.parametrize("slack", [0, 1])
@pytest.mark.parametrize("tile", TILES, ids=lambda t: f"type{t[0]:#x}_{t[1]}x{t[2]}x{t[3]}")
def test_s16_types_on_the_dot_product_kernel(gpu, oracle, tile, slack):
    lib, torch = gpu
    tf, M0, N0, K0 = tile
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=4100 + M0 + K0, slack=max(slack, 0),
                                         shapes=_shapes(M0, N0, K0))):
        if not slack and (c.lhs_offset or c.rhs_offset or c.out_offset):
            continue
        rng = np.random.default_rng(ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        if c.M and c.N and c.K:
            # (s16 x s16 with K in whole 64-element steps and more than 32 rows
            # and columns runs on the matrix cores: tests/test_gpu_s16_mfma.py)
            # (the other two from 128 rows and columns on, on a widened right-hand side)
            served = {"mmt4d_dot2"} | ({"mmt4d_mfma_128x128_s16"} if tf == uk.MMT4D_TYPE_S16S16S32
                                       else {"mmt4d_mfma_128x128_s16_widened"})
            assert lib.last_kernel_name() in served, lib.last_kernel_name()


def test_s16_tile_rows_that_are_not_a_power_of_two_stay_on_the_scalar_kernel(gpu, oracle):
    lib, torch = gpu
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S16S16S32, 4, 4, 6
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=77, shapes=((3, 2, 5),))):
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want)
        assert lib.last_kernel_name() == "mmt4d_generic"


def test_s16_full_range_products_wrap_like_int32(gpu):
    """-32768 * -32768 summed over K overflows 32 bits: the reference's int32
    accumulator wraps, and so must the dot products (no saturation)."""
    lib, torch = gpu
    M0 = N0 = 16; K0 = 2; K1 = 64
    lhs = torch.full((K1 * M0 * K0,), -32768, dtype=torch.int16, device="cuda")
    rhs = torch.full((K1 * N0 * K0,), -32768, dtype=torch.int16, device="cuda")
    out = torch.zeros(M0 * N0, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0, M0 * N0,
              1, 1, K1, M0, N0, K0, uk.MMT4D_TYPE_S16S16S32 | 0x200)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_dot2"
    want = (K1 * K0 * (1 << 30)) % (1 << 32)
    want = want - (1 << 32) if want >= (1 << 31) else want
    assert (out.cpu() == want).all()


def test_s16_negative_strides_on_device_operands(gpu, oracle):
    """Row panels walked downwards in memory (negative stride0 on all three
    operands): legal for mmt4d (the reference only does pointer arithmetic
    with them, mmt4d.c:70-83) and served by the dot-product kernel."""
    lib, torch = gpu
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S16S16S32, 8, 8, 4
    M, N, K = 5, 9, 11
    dl, dr, do = K * M0 * K0, K * N0 * K0, N * M0 * N0
    ls, rs, os_ = -(dl + 2), -(dr + 4), -(do + 3)
    rng = np.random.default_rng(9)
    lhs = rng.integers(-32768, 32768, (M - 1) * -ls + dl, dtype=np.int16)
    rhs = rng.integers(-32768, 32768, (N - 1) * -rs + dr, dtype=np.int16)
    out0 = rng.integers(-1000, 1000, (M - 1) * -os_ + do, dtype=np.int32)
    loff, roff, ooff = (M - 1) * -ls, (N - 1) * -rs, (M - 1) * -os_
    flags = tf | uk.MMT4D_ACCUMULATE | 0x200
    want = out0.copy()
    oracle.mmt4d(lhs, loff, ls, rhs, roff, rs, want, ooff, os_, M, N, K, M0, N0, K0, flags)
    d = [T.DeviceBytes(torch, a) for a in (lhs, rhs, out0)]
    lib.mmt4d(d[0].ptr, loff, ls, d[1].ptr, roff, rs, d[2].ptr, ooff, os_, M, N, K, M0, N0, K0, flags)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_dot2"
    assert np.array_equal(d[2].numpy().view(np.int32), want)
