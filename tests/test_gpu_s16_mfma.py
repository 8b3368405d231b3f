"""s16 x s16 -> s32 on the matrix cores (four 8-bit products per element pair,
row-sum correction for the biased low bytes): bit-exact, modulo 2^32, against
the oracle on FULL-RANGE inputs (every byte pattern of both halves, the
extremes -32768 and 32767 planted in every row), for the reference's x86 tile
16x16x2 (runtime/src/iree/builtins/ukernel/arch/x86_64/mmt4d_x86_64_avx512_vnni.c)
and other row widths, ragged tile counts, ACCUMULATE on and off, loose strides
and odd offsets; shapes the kernel does not serve stay on the dot-product
kernel with the same results."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

S16 = uk.MMT4D_TYPE_S16S16S32
MFMA_NAME = "mmt4d_mfma_128x128_s16"


def _full_range(rng, nbytes):
    """Full-range s16 with the extremes planted densely."""
    n = -(-nbytes // 2)
    v = rng.integers(-32768, 32768, n).astype(np.int16)
    idx = rng.integers(0, n, max(1, n // 7))
    v[idx] = rng.choice(np.array([-32768, 32767, -1, 0, 255, 256, -256, 128, -128, 127, -129], dtype=np.int16),
                        idx.size)
    return v.view(np.uint8)[:nbytes].copy()


def _buffers(c, rng):
    lhs = _full_range(rng, max(1, c.M * c.lhs_stride0 * 2))
    rhs = _full_range(rng, max(1, c.N * c.rhs_stride0 * 2))
    out = rng.integers(-2**31, 2**31, max(1, c.M * c.out_stride0), dtype=np.int64).astype(np.int32).view(np.uint8)
    return lhs, rhs, out.copy()


# (M0, N0, K0): tile rows of 2, 4, 8, 16, 32 and 128 bytes.
TILES = [(16, 16, 2), (16, 16, 1), (8, 32, 4), (16, 16, 8), (4, 8, 16), (24, 12, 2), (16, 16, 64), (1, 16, 8)]


def _shapes(M0, N0, K0):
    """Tile counts with K in whole steps of 64 elements: one block, ragged in
    both directions around the 128x128 blocking, several blocks, one step and
    several (the pipeline is unrolled by five)."""
    ks = 64 // K0 if K0 <= 64 else 1
    mb, nb = -(-128 // M0), -(-128 // N0)
    return ((-(-40 // M0), -(-40 // N0), ks), (mb, nb, 2 * ks), (mb + 1, 2 * nb + 1, 5 * ks),
            (2 * mb - 1, nb - 1, 7 * ks), (3 * mb, 2 * nb, 11 * ks))


@pytest.mark.parametrize("slack", [0, 1])
@pytest.mark.parametrize("tile", TILES, ids=lambda t: "x".join(map(str, t)))
def test_s16_on_the_matrix_cores_is_bit_exact_on_full_range_inputs(gpu, oracle, tile, slack):
    lib, torch = gpu
    M0, N0, K0 = tile
    for ci, c in enumerate(T.mmt4d_cases(S16, M0, N0, K0, seed=900 + M0 + 3 * K0, slack=slack,
                                         shapes=_shapes(M0, N0, K0))):
        rng = np.random.default_rng(1000 * slack + ci)
        lhs, rhs, out0 = _buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        print(c.label(), flush=True)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == MFMA_NAME, (c.label(), lib.last_kernel_name())
        assert np.array_equal(got, want), c.label()


def test_s16_all_minimum_values_wrap_like_int32(gpu):
    """(-32768)^2 summed over K leaves 32 bits: the reference's int32
    accumulator wraps, and so do the byte products and their recombination."""
    lib, torch = gpu
    M0 = N0 = 16; K0 = 2; M1 = N1 = 4
    for K1, fill_l, fill_r in ((64, -32768, -32768), (96, 32767, -32768), (32, 32767, 32767), (160, -32768, 255)):
        lhs = torch.full((M1 * K1 * M0 * K0,), fill_l, dtype=torch.int16, device="cuda")
        rhs = torch.full((N1 * K1 * N0 * K0,), fill_r, dtype=torch.int16, device="cuda")
        out = torch.zeros(M1 * N1 * M0 * N0, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
                  N1 * M0 * N0, M1, N1, K1, M0, N0, K0, S16 | 0x200)
        lib.synchronize()
        assert lib.last_kernel_name() == MFMA_NAME
        want = (K1 * K0 * fill_l * fill_r) % (1 << 32)
        want = want - (1 << 32) if want >= (1 << 31) else want
        assert (out.cpu() == want).all(), (K1, fill_l, fill_r)


def test_s16_shapes_outside_the_matrix_core_kernel_keep_their_results(gpu, oracle):
    """K that is not a whole number of 64-element steps, and problems of 32
    rows or columns and fewer, stay on the vector dot-product kernel."""
    lib, torch = gpu
    M0, N0, K0 = 16, 16, 2
    for ci, c in enumerate(T.mmt4d_cases(S16, M0, N0, K0, seed=5, slack=0,
                                         shapes=((4, 4, 33), (2, 8, 32), (8, 2, 64), (4, 4, 31)))):
        lhs, rhs, out0 = _buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == "mmt4d_dot2", c.label()
        assert np.array_equal(got, want), c.label()


def test_s16_matrix_core_kernel_agrees_with_the_dot_product_kernel_at_size(gpu):
    """2048 x 2048 x 4096 in the reference's 16x16x2 tiles, full-range data:
    too large for the CPU oracle in a test, so the two device kernels, which
    share no arithmetic (byte products on the matrix cores against 16-bit dot
    products on the vector ALUs), check each other bit for bit."""
    lib, torch = gpu
    M0 = N0 = 16; K0 = 2
    M1 = N1 = 128; K1 = 2048
    g = torch.Generator(device="cuda"); g.manual_seed(3)
    lhs = torch.randint(-32768, 32768, (M1 * K1 * M0 * K0,), dtype=torch.int16, device="cuda", generator=g)
    rhs = torch.randint(-32768, 32768, (N1 * K1 * N0 * K0,), dtype=torch.int16, device="cuda", generator=g)
    outs = []
    for mode in (uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_MFMA_VARIANT + 1):   # variant 1: no s16 kernel -> dot products
        lib.set_kernel_mode(mode)
        out = torch.zeros(M1 * N1 * M0 * N0, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        try:
            lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
                      N1 * M0 * N0, M1, N1, K1, M0, N0, K0, S16 | 0x200)
            lib.synchronize()
        finally:
            lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        outs.append((lib.last_kernel_name(), out))
    assert outs[0][0] == MFMA_NAME and outs[1][0] == "mmt4d_dot2", [n for n, _ in outs]
    assert torch.equal(outs[0][1], outs[1][1])


# (type, M0, N0, K0): the reference's x86 tiles for these types (16x16x2 for
# s16 x s8, 1x32x8 for s16 x u4: arch/x86_64/mmt4d_x86_64_tiles.inl) and others.
WIDENED_TILES = [(uk.MMT4D_TYPE_S16S8S32, 16, 16, 2), (uk.MMT4D_TYPE_S16S8S32, 8, 8, 16),
                 (uk.MMT4D_TYPE_S16S8S32, 24, 12, 4), (uk.MMT4D_TYPE_S16U4S32, 1, 32, 8),
                 (uk.MMT4D_TYPE_S16U4S32, 16, 16, 32), (uk.MMT4D_TYPE_S16U4S32, 4, 8, 2)]
WIDENED_NAME = "mmt4d_mfma_128x128_s16_widened"


@pytest.mark.parametrize("slack", [0, 16])
@pytest.mark.parametrize("tile", WIDENED_TILES, ids=lambda t: f"type{t[0]:#x}_{t[1]}x{t[2]}x{t[3]}")
def test_s16_by_s8_and_u4_run_on_a_widened_right_hand_side(gpu, oracle, tile, slack):
    """s16 x s8 and s16 x u4 with 128 rows and columns or more and K in whole
    steps of 64 elements: the right-hand side is widened to s16 and the s16
    matrix-core kernel runs; full-range inputs (every byte value on the RHS:
    all s8 values, both nibbles from 0 to 15), ACCUMULATE off and on, loose
    strides and offsets, bit for bit against the oracle. One row or column
    fewer, or a K remainder, stays on the dot-product kernel."""
    lib, torch = gpu
    tf, M0, N0, K0 = tile
    ks = 64 // K0
    mb, nb = -(-128 // M0), -(-128 // N0)
    shapes = ((mb, nb, ks), (mb + 1, 2 * nb + 1, 3 * ks), (2 * mb + 1, nb, 5 * ks))
    rhs_bits = 8 if tf == uk.MMT4D_TYPE_S16S8S32 else 4
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=300 + M0 + K0, slack=slack, shapes=shapes)):
        rng = np.random.default_rng(7000 + 100 * slack + ci)
        lhs = _full_range(rng, max(1, (c.M * c.lhs_stride0 + c.lhs_offset) * 2 + 64))
        rhs = rng.integers(0, 256, (c.N * c.rhs_stride0 + c.rhs_offset) * rhs_bits // 8 + 64, dtype=np.uint8)
        out0 = rng.integers(-2**31, 2**31, c.M * c.out_stride0 + c.out_offset + 16,
                            dtype=np.int64).astype(np.int32).view(np.uint8).copy()
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert lib.last_kernel_name() == WIDENED_NAME, (c.label(), lib.last_kernel_name())
        assert np.array_equal(got, want), c.label()
    if M0 > 1:
        for shape in ((mb - 1, nb, ks), (mb, nb, ks + 1)):
            c = next(iter(T.mmt4d_cases(tf, M0, N0, K0, seed=5, slack=0, shapes=(shape,))))
            rng = np.random.default_rng(31)
            lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
            want = out0.copy()
            G.run_mmt4d_case(oracle, c, lhs, rhs, want)
            got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
            assert lib.last_kernel_name() == "mmt4d_dot2", (shape, lib.last_kernel_name())
            assert np.array_equal(got, want), c.label()
