"""Tile rows under 16 bytes in shapes the matrix-core kernels do not take as
they are - one-byte rows (s8 8x8x1, arm64's tile without dot-product
instructions: arch/arm_64/mmt4d_arm_64_tiles.inl), rows of 2, 4 or 8 bytes in
tiles whose height is not a multiple of the rows a 16-byte piece spans, f8 rows
under 16 bytes: both operands are regrouped along K into 16-byte rows first.
Against the oracle, bit for bit (integers; floats on the reference's test
values, whose sums are exact in any order), ACCUMULATE off and on, loose
strides and offsets, K with a remainder that the last regrouped tile fills up
with zeros."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

TILES = [(uk.MMT4D_TYPE_S8S8S32, 8, 8, 1), (uk.MMT4D_TYPE_S8S8S32, 4, 16, 2), (uk.MMT4D_TYPE_S8S8S32, 5, 3, 4),
         (uk.MMT4D_TYPE_S8S8S32, 1, 16, 8), (uk.MMT4D_TYPE_F16F16F32, 4, 4, 1), (uk.MMT4D_TYPE_BF16BF16F32, 2, 8, 2),
         (uk.MMT4D_TYPE_F32F32F32, 2, 6, 1), (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 8),
         (uk.MMT4D_TYPE_S16S16S32, 4, 4, 1),
         (uk.MMT4D_TYPE_F16F16F16 | uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS, 2, 8, 2)]


@pytest.mark.parametrize("tile", TILES, ids=lambda t: f"type{t[0]:#x}_{t[1]}x{t[2]}x{t[3]}")
def test_declined_narrow_tiles_run_regrouped(gpu, oracle, tile):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    tf, M0, N0, K0 = tile
    assert not lib.mmt4d_info(M0, N0, K0, tf)           # not advertised: callers pass the fallback flag
    tf, extra = tf & 0xFF, tf & ~0xFF
    mb, nb = -(-256 // M0), -(-256 // N0)
    s16 = tf == uk.MMT4D_TYPE_S16S16S32
    # K elements: with and without a remainder (the s16 kernel needs whole steps of 64 elements)
    ks = (256 // K0, 320 // K0) if s16 else (256 // K0, (300 + K0 - 1) // K0)
    shapes = ((mb, nb, ks[0]), (mb + 1, nb + 2, ks[1]))
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=50 + M0 + K0, slack=16, shapes=shapes,
                                         extra_flags=extra)):
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(600 + ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == "mmt4d_mfma_retiled", (c.label(), lib.last_kernel_name())
        assert np.array_equal(got, want), c.label()
    # a small problem is not worth the two extra passes: the scalar kernel (or, for s16, vector dot products)
    c = next(iter(T.mmt4d_cases(tf, M0, N0, K0, seed=3, slack=0, shapes=((2, 2, 8),), extra_flags=extra)))
    lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(1))
    want = out0.copy()
    G.run_mmt4d_case(oracle, c, lhs, rhs, want)
    got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
    assert lib.last_kernel_name() in ("mmt4d_generic", "mmt4d_dot2"), lib.last_kernel_name()
    assert np.array_equal(got, want), c.label()


def test_s8s4_two_element_rows_in_four_row_tiles(gpu, oracle):
    """arm64's s8 x s4 tile Mx16x2 (arch/arm_64/mmt4d_arm_64_base.c:296) from
    512 rows on: the s8 kernels do not take 4x16x2, so both operands are
    regrouped along K, the weights widened on the way."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S8S4S32, 4, 16, 2
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=77, slack=16,
                                         shapes=((128, 3, 40), (131, 9, 75)))):
        rng = np.random.default_rng(ci)
        lhs = rng.integers(-128, 128, c.M * c.lhs_stride0 + c.lhs_offset + 64, dtype=np.int8).view(np.uint8)
        rhs = rng.integers(0, 256, (c.N * c.rhs_stride0 + c.rhs_offset) // 2 + 64, dtype=np.uint8)
        out0 = rng.integers(-2 ** 31, 2 ** 31, c.M * c.out_stride0 + c.out_offset + 16,
                            dtype=np.int64).astype(np.int32).view(np.uint8)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == "mmt4d_mfma_s8s4_expanded", (c.label(), lib.last_kernel_name())
        assert np.array_equal(got, want), c.label()
