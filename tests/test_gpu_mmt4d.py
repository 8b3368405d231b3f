"""GPU parity of iree_uk_mmt4d against the CPU oracle, through the C-ABI.
Integer types: bit-exact. Float types: bit-exact on the small-integer inputs
of the reference's own tests (every partial sum is exact, so the summation
order does not matter), and within the stated tolerance on N(0,1) inputs:
max|gpu-ref| / max|ref| <= 1e-2 for f16/bf16 and <= 2e-2 for f8, against the
f32-accumulating oracle."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

TOL = {uk.MMT4D_TYPE_F16F16F32: 1e-2, uk.MMT4D_TYPE_BF16BF16F32: 1e-2,
       uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: 2e-2, uk.MMT4D_TYPE_F32F32F32: 1e-5}


@pytest.fixture(autouse=True)
def _reset_modes(lib):
    yield
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_pointer_mode(uk.POINTER_MODE_AUTO)


@pytest.mark.parametrize("mode", [uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_GENERIC])
@pytest.mark.parametrize("n", range(len(G.MMT4D_TILES)))
def test_mmt4d_reference_test_grid(gpu, oracle, n, mode):
    """tools/mmt4d_test.c's grid: every type triple, odd tile shapes,
    degenerate M/N/K, ACCUMULATE on/off, loose strides, non-zero offsets;
    memcmp over the whole output buffer."""
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    tf, M0, N0, K0, extra = G.MMT4D_TILES[n]
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=13000 + n, extra_flags=extra)):
        rng = np.random.default_rng(ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())


# (type, M0, N0, K0) served by the MFMA kernels, with tile-count shapes that
# cover: single tile, ragged against the workgroup tile in M and N, K both
# below and above one pipeline step, and a several-workgroup case.
MFMA_TILES = [
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 2), (uk.MMT4D_TYPE_S8S8S32, 32, 16, 8),
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 16), (uk.MMT4D_TYPE_S8S8S32, 16, 16, 64),
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 4), (uk.MMT4D_TYPE_S8S8S32, 16, 16, 8),
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 32), (uk.MMT4D_TYPE_S8S8S32, 8, 8, 2),
    (uk.MMT4D_TYPE_S8S8S32, 8, 32, 4), (uk.MMT4D_TYPE_S8S8S32, 64, 16, 1),
    (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16), (uk.MMT4D_TYPE_F16F16F32, 16, 16, 1),
    (uk.MMT4D_TYPE_F16F16F32, 16, 16, 8), (uk.MMT4D_TYPE_F16F16F32, 8, 16, 4),
    (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 2), (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 8),
    (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 32),
    (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 32),
    (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 16),
    (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 128),
    (uk.MMT4D_TYPE_F32F32F32, 16, 16, 1), (uk.MMT4D_TYPE_F32F32F32, 16, 16, 4),
    (uk.MMT4D_TYPE_F32F32F32, 8, 8, 2), (uk.MMT4D_TYPE_F32F32F32, 16, 16, 32),
    # tile heights that do not divide the workgroup tiles (a partial panel at
    # the end of each block), with regrouping and with direct loaders
    (uk.MMT4D_TYPE_S8S8S32, 24, 16, 4), (uk.MMT4D_TYPE_S8S8S32, 16, 24, 2),
    (uk.MMT4D_TYPE_F16F16F32, 24, 48, 2), (uk.MMT4D_TYPE_S8S8S32, 40, 24, 16),
    (uk.MMT4D_TYPE_BF16BF16F32, 12, 20, 4), (uk.MMT4D_TYPE_F32F32F32, 24, 40, 1),
]


def _mfma_shapes(M0, N0, K0, bits):
    kb = K0 * bits // 8  # bytes of K per tile row
    k_small = max(1, 32 // kb)
    k_big = max(3, 700 // kb)          # several pipeline steps plus a remainder
    k_whole = max(1, 5 * 128 // kb)    # a whole number of steps, odd count
    m_wg = max(1, 256 // M0)
    n_wg = max(1, 256 // N0)
    return ((1, 1, 1), (1, 1, k_small), (2, 3, k_big), (m_wg + 1, 1, k_small + 1),
            (1, n_wg + 3, 5), (m_wg + 2, n_wg + 1, k_big // 2 + 1), (0, 2, 2),
            (2, 2, 0), (m_wg + 1, 2 * n_wg + 1, k_whole), (3, 2, 2 * k_whole))


# 0 = let the library choose by problem size; 1..4 = force the 256x256,
# 128x128, 64x64 and M-thin workgroup shapes (a forced shape that cannot serve
# a case falls through to the next one that can; 4 is the barrier-free thin
# kernel when K is a whole number of 64-byte steps and rows are at least 8
# bytes wide, else the 32x64 kernel through LDS: the shapes below have both;
# 5 is the thin kernel on the transposed problem and 6 the same kernel with
# 64x64 blocks, under the same conditions; 7 is the 256x128 shape, 8 the
# 128x512 shape; 11 is the 64x64 shape with the deep pipeline, 12 .. 15 are
# the narrow-row kernels in the 256x256 / 128x512 / 128x128 / 64x64 shape, which
# serve tile rows of 2 or 4 bytes with N0 = 16 and hand everything else on, and
# 16 .. 20 the LDS-direct ping-pong pipeline in the 256x256 / 128x512 / 128x128 /
# 64x64 / 256x128 shape).
# Tile rows of one byte (s8, K0 = 1) have no MFMA kernel: iree_uk_mmt4d_info
# says so and the reference grid above covers them on the scalar kernel. The
# entry stays in the list, named for what it is, and is asserted unserved.
def _tile_id(n):
    tf, M0, N0, K0 = MFMA_TILES[n]
    name = f"{n}-type{tf:#x}_{M0}x{N0}x{K0}"
    return name + "_one_byte_rows_have_no_mfma_kernel" if (tf, K0) == (uk.MMT4D_TYPE_S8S8S32, 1) else name


def _variant_applies(n, variant):
    """Forced shapes that a tile cannot take hand the call on to the choice by
    size, i.e. repeat variant 0: the deep 64x64 pipeline (11) exists for tile
    rows under 16 bytes, the narrow-row kernels (12 .. 15) for rows of 2 or 4
    bytes with N0 = 16, the LDS-direct pipeline (16 .. 20): its small shapes (18,
    19) not for the 8-bit floats, its 256x128 shape (20) for rows of 16 bytes and more."""
    tf, M0, N0, K0 = MFMA_TILES[n]
    row_bytes = K0 * uk.MMT4D_TYPE_BITS[tf][0] // 8
    if variant == 11:
        return row_bytes < 16
    if variant in (12, 13, 14, 15):
        return row_bytes in (2, 4) and N0 == 16
    if variant in (18, 19):
        # the LDS-direct pipeline in its small shapes: one 16-byte piece per lane operand (not the 8-bit floats)
        return tf != uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32
    if variant == 20:
        return row_bytes >= 16
    return True


_TILE_VARIANTS = [pytest.param(n, v, id=f"{_tile_id(n)}-{v}")
                  for n in range(len(MFMA_TILES))
                  for v in (0, 1, 2, 3, 4, 5, 6, 7, 8, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20) if _variant_applies(n, v)]


_EXACT_CASES = {}   # (tile index, case index) -> (lhs, rhs, initial out, oracle result)


@pytest.mark.parametrize("n,variant", _TILE_VARIANTS)
def test_mmt4d_mfma_shapes_exact_inputs(gpu, oracle, n, variant):
    lib, torch = gpu
    tf, M0, N0, K0 = MFMA_TILES[n]
    if (tf, K0) == (uk.MMT4D_TYPE_S8S8S32, 1):
        assert not lib.mmt4d_info(M0, N0, K0, tf)
        return
    assert lib.mmt4d_info(M0, N0, K0, tf)
    lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
    bits = uk.MMT4D_TYPE_BITS[tf][0]
    # Loose strides and offsets in steps of 16 elements (one-element slack on
    # the matrix-core kernels has a test of its own below).
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=14000 + n, slack=16,
                                         shapes=_mfma_shapes(M0, N0, K0, bits))):
        # The inputs and the oracle's answer depend on the tile and the case, not
        # on the forced variant: computed once per tile, reused by every variant.
        key = (n, ci)
        if key not in _EXACT_CASES:
            rng = np.random.default_rng(ci)
            lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
            want = out0.copy()
            G.run_mmt4d_case(oracle, c, lhs, rhs, want)
            _EXACT_CASES[key] = (lhs, rhs, out0, want)
        lhs, rhs, out0, want = _EXACT_CASES[key]
        out0 = out0.copy()
        # No generic-fallback flag: only an MFMA kernel may serve these calls.
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        if c.M and c.N and c.K:  # K == 0 is a zero fill, left to the generic kernel
            assert lib.last_kernel_name().startswith("mmt4d_mfma"), lib.last_kernel_name()


# Shapes big enough for the 256x256 variant whose last row and/or column of
# workgroups is mostly padding: the library computes those as separate strips
# with the smaller variants. (tile counts M1, N1, K1 for 16x16x16 s8 tiles)
@pytest.mark.parametrize("shape", [(256, 257, 4), (241, 273, 5), (257, 256, 8)])
def test_mmt4d_split_off_remainder_strips(gpu, oracle, shape):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S8S8S32, 16, 16, 16
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=777, slack=16, shapes=(shape,))):
        rng = np.random.default_rng(100 + ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        assert lib.last_kernel_name().startswith(("mmt4d_mfma_256x256", "mmt4d_mfma_128x512")), lib.last_kernel_name()


# 16-bit float outputs: an MFMA kernel serves them when the caller allows a
# single rounding at the end (SKIP_INTERMEDIATE_ROUNDINGS); on the reference
# tests' small-integer inputs every f32 partial sum is exact, so the result must
# equal the oracle's bit for bit, final rounding included.
@pytest.mark.parametrize("variant", [0, 1, 3, 4, 5, 8, 16])
@pytest.mark.parametrize("tf,M0,N0,K0", [
    (uk.MMT4D_TYPE_F16F16F16, 16, 16, 8), (uk.MMT4D_TYPE_F16F16F16, 16, 16, 1),
    (uk.MMT4D_TYPE_BF16BF16BF16, 16, 16, 8), (uk.MMT4D_TYPE_BF16BF16BF16, 8, 32, 2)])
def test_mmt4d_16bit_outputs_single_rounding(gpu, oracle, tf, M0, N0, K0, variant):
    lib, torch = gpu
    assert lib.mmt4d_info(M0, N0, K0, tf | uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS)
    assert not lib.mmt4d_info(M0, N0, K0, tf)   # rounding after every element: generic only
    lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=15000, slack=16,
                                         extra_flags=uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS,
                                         shapes=_mfma_shapes(M0, N0, K0, 16))):
        rng = np.random.default_rng(ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        if c.M and c.N and c.K:
            assert lib.last_kernel_name().startswith("mmt4d_mfma"), lib.last_kernel_name()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 8, 16, 17, 18, 19])
@pytest.mark.parametrize("tf", [uk.MMT4D_TYPE_F16F16F16, uk.MMT4D_TYPE_BF16BF16BF16])
def test_mmt4d_16bit_outputs_round_once_when_k_has_a_remainder(gpu, oracle, tf, variant):
    """Sums that no longer fit a 16-bit float exactly (small-integer inputs, a
    long K, ACCUMULATE) with K a few tiles past a whole number of pipeline
    steps: the result is rounded once, after all of K, whatever kernel is
    forced. A library that ran the remainder of K as a second launch on top of
    the rounded result of the first would differ in some elements."""
    lib, torch = gpu
    M0, N0, K0 = 24, 64, 4
    flags = tf | uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS | uk.MMT4D_ACCUMULATE
    lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
    for seed, (M, N, K) in enumerate(((12, 3, 130), (5, 9, 259), (11, 4, 33))):
        c = T.Mmt4dCase(flags, M, N, K, M0, N0, K0, K * M0 * K0 + 16, K * N0 * K0, N * M0 * N0 + 16, 16, 0, 0)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(99 + seed))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        assert lib.last_kernel_name().startswith("mmt4d_mfma"), lib.last_kernel_name()
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)


def test_mmt4d_single_row_tiles_equal_row_major_matmul(gpu):
    """With M0 = N0 = 1 the mmt4d layouts are plain row-major [M][K], [N][K]
    and [M][N]: the call must equal the integer matrix product A . B^T
    (independent of the oracle: a closed form)."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    rng = np.random.default_rng(3)
    for (M, N, K, K0) in ((300, 260, 512, 16), (257, 131, 192, 64), (64, 64, 64, 16)):
        a = rng.integers(-128, 128, (M, K), dtype=np.int8)
        bt = rng.integers(-128, 128, (N, K), dtype=np.int8)
        out0 = rng.integers(-1000, 1000, (M, N)).astype(np.int32)
        d = [T.DeviceBytes(torch, x) for x in (a, bt, out0)]
        flags = uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE
        lib.mmt4d(d[0].ptr, 0, K, d[1].ptr, 0, K, d[2].ptr, 0, N, M, N, K // K0, 1, 1, K0, flags)
        lib.synchronize()
        assert lib.last_kernel_name().startswith("mmt4d_mfma"), lib.last_kernel_name()
        want = out0.astype(np.int64) + a.astype(np.int64) @ bt.astype(np.int64).T
        got = d[2].numpy().view(np.int32).reshape(M, N)
        assert np.array_equal(got, want.astype(np.int32)), (M, N, K, K0)


def _normal_operand(rng, kind, n, scale=1.0):
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    if kind == "f16":
        return x.astype(np.float16).view(np.uint16)
    if kind == "bf16":
        return T.f32_to_bf16_bits(x)
    if kind == "f8":
        x = x * (448.0 / np.abs(x).max())
        return T.f32_to_f8e4m3fn_bits(x)
    return x


@pytest.mark.parametrize("tf,M0,N0,K0", [
    (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16), (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 2),
    (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 8),
    (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 32),
    (uk.MMT4D_TYPE_F32F32F32, 8, 8, 4), (uk.MMT4D_TYPE_F32F32F32, 16, 16, 1)])
@pytest.mark.parametrize("accumulate", [0, 1])
@pytest.mark.parametrize("variant", [0, 1, 8, 16, 17])
def test_mmt4d_float_tolerance_on_normal_inputs(gpu, oracle, tf, M0, N0, K0, accumulate, variant):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
    lk = T.MMT4D_KINDS[tf][0]
    rng = np.random.default_rng(21)
    M, N, K = 9, 11, max(1, 2048 // K0)
    lhs = _normal_operand(rng, lk, M * K * M0 * K0)
    rhs = _normal_operand(rng, lk, N * K * N0 * K0)
    out0 = rng.standard_normal(M * N * M0 * N0).astype(np.float32) * 10
    flags = tf | 0x200 | (uk.MMT4D_ACCUMULATE if accumulate else 0)
    want = out0.copy()
    oracle.mmt4d(lhs, 0, K * M0 * K0, rhs, 0, K * N0 * K0, want, 0, N * M0 * N0,
                 M, N, K, M0, N0, K0, flags)
    d = [T.DeviceBytes(torch, a) for a in (lhs, rhs, out0)]
    lib.mmt4d(d[0].ptr, 0, K * M0 * K0, d[1].ptr, 0, K * N0 * K0, d[2].ptr, 0,
              N * M0 * N0, M, N, K, M0, N0, K0, flags)
    lib.synchronize()
    got = d[2].numpy().view(np.float32)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= TOL[tf], (err, lib.last_kernel_name())


def test_mmt4d_host_pointers_are_staged(gpu, oracle):
    lib, torch = gpu
    for ci, c in enumerate(T.mmt4d_cases(uk.MMT4D_TYPE_S8S8S32, 16, 16, 2, seed=41,
                                         shapes=((2, 3, 5), (1, 1, 0), (5, 7, 13)))):
        rng = np.random.default_rng(ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = out0.copy()
        lib.mmt4d(lhs.ctypes.data - c.lhs_offset, c.lhs_offset, c.lhs_stride0,
                  rhs.ctypes.data - c.rhs_offset, c.rhs_offset, c.rhs_stride0,
                  got.ctypes.data - c.out_offset * 4, c.out_offset, c.out_stride0,
                  c.M, c.N, c.K, c.M0, c.N0, c.K0, c.flags | 0x200)
        assert np.array_equal(got, want), c.label()


def _pow2_bits(tf, exponent: int) -> int:
    """Bit pattern of 2**exponent as an f16 or bf16 element (subnormals included)."""
    if tf in (uk.MMT4D_TYPE_F16F16F32, uk.MMT4D_TYPE_F16F16F16):
        return int(np.float16(2.0 ** exponent).view(np.uint16))
    return int(np.float32(2.0 ** exponent).view(np.uint32) >> 16)


@pytest.mark.parametrize("tf,sub_e,big_e", [(uk.MMT4D_TYPE_F16F16F32, -20, 10),
                                             (uk.MMT4D_TYPE_BF16BF16F32, -130, 100)])
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 8, 16])
def test_mmt4d_subnormal_inputs_matrix_cores_keep_scalar_kernel_flushes(gpu, oracle, tf, sub_e, big_e, variant):
    """Pins how subnormal f16 / bf16 inputs are read. The reference's generic
    tile functions flush them to zero (common.h:664-700), and so do the oracle
    and the scalar kernel, bit for bit. The matrix-core kernels keep them, as
    the instruction does (and as the reference's own AVX-512 f16 tile function
    does through vcvtph2ps). Powers of two keep every product and sum exact, so
    both expectations are exact: LHS = one subnormal value, RHS = one large
    value, each output K*K0 products."""
    lib, torch = gpu
    M0 = N0 = K0 = 16
    M, N, K = (1, 8, 8) if variant == 4 else (32, 32, 8)
    lhs = np.full(M * K * M0 * K0, _pow2_bits(tf, sub_e), dtype=np.uint16)
    rhs = np.full(N * K * N0 * K0, _pow2_bits(tf, big_e), dtype=np.uint16)
    out0 = np.zeros(M * N * M0 * N0, dtype=np.float32)
    flags = tf | 0x200
    flushed = out0.copy()
    oracle.mmt4d(lhs, 0, K * M0 * K0, rhs, 0, K * N0 * K0, flushed, 0, N * M0 * N0, M, N, K, M0, N0, K0, flags)
    assert not flushed.any()          # the reference semantics: every product is 0 * big
    kept = np.full_like(out0, np.float32(K * K0 * 2.0 ** (sub_e + big_e)))
    d = [T.DeviceBytes(torch, a) for a in (lhs, rhs, out0)]
    for mode, want, prefix in ((uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO,
                                kept, "mmt4d_mfma"),
                               (uk.KERNEL_MODE_GENERIC, flushed, "mmt4d_generic")):
        lib.set_kernel_mode(mode)
        try:
            lib.mmt4d(d[0].ptr, 0, K * M0 * K0, d[1].ptr, 0, K * N0 * K0, d[2].ptr, 0, N * M0 * N0,
                      M, N, K, M0, N0, K0, flags)
            lib.synchronize()
        finally:
            lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        assert lib.last_kernel_name().startswith(prefix), lib.last_kernel_name()
        assert np.array_equal(d[2].numpy().view(np.float32), want), lib.last_kernel_name()


def _pitch(mode: int, dense: int) -> int:
    """Row pitches a dense 2-D copy cannot express: 0 loose, 1 negative,
    2 zero (broadcast), 3 / 4 shorter than a row (overlapping rows), + and -."""
    return {0: dense + 2, 1: -(dense + 2), 2: 0, 3: dense // 2, 4: -(dense // 2)}[mode]


@pytest.mark.parametrize("tf,M0,N0,K0", [(uk.MMT4D_TYPE_S8S8S32, 16, 16, 16),
                                         (uk.MMT4D_TYPE_S8S8S32, 16, 16, 2),
                                         (uk.MMT4D_TYPE_S16S16S32, 8, 8, 2)])
def test_mmt4d_host_operands_with_negative_zero_and_overlapping_pitches(gpu, oracle, tf, M0, N0, K0):
    """Strides that are legal for mmt4d (the reference only does pointer
    arithmetic with them, mmt4d.c:70-83) survive the staging of host operands:
    negative (rows walked downwards), zero (every row panel the same memory)
    and shorter than a row; the output with a negative stride."""
    lib, torch = gpu
    lb, rb, ob = uk.MMT4D_TYPE_BITS[tf]
    M, N, K = 3, 5, 8
    dl, dr, dout = K * M0 * K0, K * N0 * K0, N * M0 * N0
    rng = np.random.default_rng(77)
    before = lib.staging_bytes()
    for lm in range(5):
        for rm in range(5):
            for om in (0, 1):
                ls, rs, os_ = _pitch(lm, dl), _pitch(rm, dr), _pitch(om, dout)
                loff, roff, ooff = (max(0, -(M - 1) * ls), max(0, -(N - 1) * rs), max(0, -(M - 1) * os_))
                lhs = rng.integers(0, 256, ((M - 1) * abs(ls) + dl) * lb // 8, dtype=np.uint8)
                rhs = rng.integers(0, 256, ((N - 1) * abs(rs) + dr) * rb // 8, dtype=np.uint8)
                out0 = rng.integers(0, 256, ((M - 1) * abs(os_) + dout) * ob // 8, dtype=np.uint8)
                flags = tf | (uk.MMT4D_ACCUMULATE if (lm + rm) & 1 else 0) | 0x200
                want = out0.copy()
                oracle.mmt4d(lhs, loff, ls, rhs, roff, rs, want, ooff, os_, M, N, K, M0, N0, K0, flags)
                got = out0.copy()
                lib.mmt4d(lhs.ctypes.data, loff, ls, rhs.ctypes.data, roff, rs, got.ctypes.data, ooff, os_,
                          M, N, K, M0, N0, K0, flags)
                assert np.array_equal(got, want), (lm, rm, om, lib.last_kernel_name())
    # The copies came out of the thread's arena: it grew at most once per size
    # class, not once per call, and can be handed back.
    held = lib.staging_bytes()
    assert held >= before and held > 0
    assert lib.release_staging() == 0 and lib.staging_bytes() == 0


def test_thread_local_device_memory_is_released_when_the_thread_ends(gpu):
    """The staging arena (host operands) and the K-split workspace belong to the
    calling thread and go back to the device when it ends: a pool of
    short-lived threads must not leak device memory."""
    import threading
    lib, torch = gpu
    torch.cuda.synchronize()
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S8S8S32, 16, 16, 16
    M, N, K = 64, 256, 256                     # 4 MiB + 16 MiB of operands, 4 MiB of result
    rng = np.random.default_rng(5)
    lhs = rng.integers(-128, 128, M * K * M0 * K0, dtype=np.int8)
    rhs = rng.integers(-128, 128, N * K * N0 * K0, dtype=np.int8)
    held = []

    def work():
        out = np.zeros(M * N * M0 * N0, dtype=np.int32)
        lib.mmt4d(lhs.ctypes.data, 0, K * M0 * K0, rhs.ctypes.data, 0, K * N0 * K0, out.ctypes.data, 0,
                  N * M0 * N0, M, N, K, M0, N0, K0, tf)
        held.append((lib.staging_bytes(), int(out[0])))

    def run_threads(n):
        for _ in range(n):
            t = threading.Thread(target=work)
            t.start()
            t.join()
        torch.cuda.synchronize()

    # The HIP runtime takes and returns device memory in chunks of its own (64 MiB
    # at a time, whenever it pleases on a fresh machine), so the check is made
    # against what a leak would cost: sixteen threads that each stage 24 MiB and
    # more would leave 384 MiB behind; a quarter of that is the limit.
    run_threads(2)
    free_before = torch.cuda.mem_get_info()[0]
    run_threads(16)
    free_after = torch.cuda.mem_get_info()[0]
    assert all(h[0] >= 24 << 20 for h in held), held          # each thread staged its own copy
    assert len({h[1] for h in held}) == 1
    assert free_before - free_after < (96 << 20), (free_before, free_after)


def test_entry_points_from_concurrent_threads(gpu, oracle):
    """The entry points are re-entrant (runtime/src/iree/builtins/ukernel/
    README.md:26): four host threads, each on its own slab of one problem
    selected through offsets (as the CPU task system slices work), one using
    host buffers (staged), the others device buffers on their own streams."""
    import threading
    lib, torch = gpu
    rng = np.random.default_rng(11)
    M1, N1, K1, M0, N0, K0 = 8, 6, 24, 16, 16, 16
    lhs = rng.integers(-128, 128, M1 * K1 * M0 * K0, dtype=np.int8)
    rhs = rng.integers(-128, 128, N1 * K1 * N0 * K0, dtype=np.int8)
    out0 = rng.integers(-99, 99, M1 * N1 * M0 * N0).astype(np.int32)
    flags = uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE | 0x200
    want = out0.copy()
    oracle.mmt4d(lhs, 0, K1 * M0 * K0, rhs, 0, K1 * N0 * K0, want, 0, N1 * M0 * N0,
                 M1, N1, K1, M0, N0, K0, flags)
    got_host = out0.copy()
    d_lhs, d_rhs, d_out = (T.DeviceBytes(torch, x) for x in (lhs, rhs, out0))
    errors = []

    def slab(t, rows):
        try:
            lo = t * rows
            if t == 0:   # host pointers, default stream
                lib.mmt4d(lhs.ctypes.data, lo * K1 * M0 * K0, K1 * M0 * K0, rhs.ctypes.data, 0,
                          K1 * N0 * K0, got_host.ctypes.data, lo * N1 * M0 * N0, N1 * M0 * N0,
                          rows, N1, K1, M0, N0, K0, flags)
            else:
                s = torch.cuda.Stream()
                lib.set_stream(s.cuda_stream)
                lib.mmt4d(d_lhs.ptr, lo * K1 * M0 * K0, K1 * M0 * K0, d_rhs.ptr, 0, K1 * N0 * K0,
                          d_out.ptr, lo * N1 * M0 * N0, N1 * M0 * N0, rows, N1, K1, M0, N0, K0,
                          flags)
                lib.synchronize()
                lib.set_stream(None)
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))

    rows = M1 // 4
    threads = [threading.Thread(target=slab, args=(t, rows)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    tile_row = N1 * M0 * N0
    got_dev = d_out.numpy().view(np.int32)
    assert np.array_equal(got_host[:rows * tile_row], want[:rows * tile_row])
    assert np.array_equal(got_host[rows * tile_row:], out0[rows * tile_row:])   # other slabs untouched
    assert np.array_equal(got_dev[rows * tile_row:], want[rows * tile_row:])
    assert np.array_equal(got_dev[:rows * tile_row], out0[:rows * tile_row])


@pytest.mark.parametrize("mode", [uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_GENERIC,
                                  uk.KERNEL_MODE_MFMA_VARIANT + 1])
@pytest.mark.parametrize("tf,M0,N0,K0", [
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 16), (uk.MMT4D_TYPE_S8S8S32, 16, 16, 2),
    (uk.MMT4D_TYPE_S8S8S32, 8, 32, 4), (uk.MMT4D_TYPE_F16F16F32, 16, 16, 8),
    (uk.MMT4D_TYPE_F32F32F32, 16, 16, 1), (uk.MMT4D_TYPE_S16S16S32, 4, 6, 3)])
def test_fused_mmt4d_unpack_equals_the_two_calls(gpu, oracle, tf, M0, N0, K0, mode):
    """iree_uk_amd_mmt4d_unpack == mmt4d into a tiled temporary + unpack of it,
    bit for bit (inputs are the reference tests' small integers, so every f32
    partial sum is exact), including ragged sizes, loose row pitch, a nonzero
    offset, ACCUMULATE, and bytes outside the matrix left untouched."""
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    lk, rk, ok = T.MMT4D_KINDS[tf]
    unpack_tf = uk.UNPACK_TYPE_I32I32 if ok == "s32" else uk.UNPACK_TYPE_F32F32
    shapes = [(3, 2, 5, 0, 0), (17, 18, 9, 5, 3), (1, 1, 1, 0, 15), (33, 5, 40, 15, 0)]
    for si, (M1, N1, K1, cut0, cut1) in enumerate(shapes):
        for acc in (0, 1):
            rows, cols = M1 * M0 - min(cut0, M0 - 1), N1 * N0 - min(cut1, N0 - 1)
            pitch, off = cols + 16 * (si % 2), 16 * ((si + acc) % 2)
            c = T.Mmt4dCase(tf | 0x200 | (uk.MMT4D_ACCUMULATE if acc else 0), M1, N1, K1, M0, N0,
                            K0, K1 * M0 * K0, K1 * N0 * K0, N1 * M0 * N0, 0, 0, 0)
            rng = np.random.default_rng(100 * si + acc)
            lhs, rhs, _ = T.make_mmt4d_buffers(c, rng)
            out0 = rng.integers(-9, 9, off + rows * pitch).astype(np.int32)
            if ok != "s32":
                out0 = out0.astype(np.float32).view(np.int32)
            # oracle: pack the accumulator matrix, mmt4d, unpack
            tiled = np.zeros(M1 * N1 * M0 * N0, np.int32)
            if acc:
                oracle.pack(out0, off, pitch, 1, tiled, 0, N1 * M0 * N0, M0 * N0, rows, cols,
                            M1, N1, M0, N0, 0, uk.PACK_TYPE_I32I32)
            G.run_mmt4d_case(oracle, c, lhs, rhs, tiled.view(np.uint8))
            want = out0.copy()
            oracle.unpack(tiled, 0, N1 * M0 * N0, M0 * N0, want, off, pitch, 1, M1, N1, M0, N0,
                          rows, cols, unpack_tf)
            d = [T.DeviceBytes(torch, x) for x in (lhs, rhs, out0)]
            lib.mmt4d_unpack(d[0].ptr, 0, c.lhs_stride0, d[1].ptr, 0, c.rhs_stride0, d[2].ptr, off,
                             pitch, rows, cols, M1, N1, K1, M0, N0, K0, c.flags)
            lib.synchronize()
            got = d[2].numpy().view(np.int32)
            assert np.array_equal(got, want), (tf, M0, N0, K0, M1, N1, K1, acc, lib.last_kernel_name())
            # host pointers (staged) give the same
            host = out0.copy()
            lib.mmt4d_unpack(lhs.ctypes.data, 0, c.lhs_stride0, rhs.ctypes.data, 0, c.rhs_stride0,
                             host.ctypes.data, off, pitch, rows, cols, M1, N1, K1, M0, N0, K0,
                             c.flags)
            assert np.array_equal(host, want)


@pytest.mark.parametrize("accumulate", [0, 1])
def test_fused_mmt4d_unpack_with_remainder_strips(gpu, accumulate):
    """A shape large enough for the 256x256 variant and ragged against it in M
    and N (so the strips are split off), with a K remainder: the fused call
    must equal mmt4d + unpack on the GPU (both halves are pinned against the
    oracle by the tests above) and, on a sample of rows, the integer product."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, K1, M0, N0, K0 = 241, 273, 5, 16, 16, 16
    rows, cols = M1 * M0 - 3, N1 * N0 - 5
    g = torch.Generator(device="cuda"); g.manual_seed(7)
    lhs = torch.randint(-128, 128, (M1, K1, M0, K0), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1, K1, N0, K0), generator=g, device="cuda", dtype=torch.int8)
    init = torch.randint(-1000, 1000, (rows, cols), generator=g, device="cuda", dtype=torch.int32)
    flags = uk.MMT4D_TYPE_S8S8S32 | (uk.MMT4D_ACCUMULATE if accumulate else 0)
    # the two reference calls (accumulator packed first when accumulating)
    tiled = torch.zeros(M1 * N1 * M0 * N0, device="cuda", dtype=torch.int32)
    if accumulate:
        lib.pack(init.data_ptr(), 0, cols, 1, tiled.data_ptr(), 0, N1 * M0 * N0, M0 * N0, rows, cols,
                 M1, N1, M0, N0, 0, uk.PACK_TYPE_I32I32)
    lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, tiled.data_ptr(), 0,
              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags)
    assert lib.last_kernel_name().startswith(("mmt4d_mfma_256x256", "mmt4d_mfma_128x512"))
    want = init.clone()
    lib.unpack(tiled.data_ptr(), 0, N1 * M0 * N0, M0 * N0, want.data_ptr(), 0, cols, 1, M1, N1, M0, N0,
               rows, cols, uk.UNPACK_TYPE_I32I32)
    got = init.clone()
    lib.mmt4d_unpack(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, got.data_ptr(),
                     0, cols, rows, cols, M1, N1, K1, M0, N0, K0, flags)
    assert lib.last_kernel_name().startswith(("mmt4d_mfma_256x256", "mmt4d_mfma_128x512"))
    lib.synchronize()
    assert torch.equal(got, want)
    # closed form on the last rows (they cross the row strip)
    a = lhs.permute(0, 2, 1, 3).reshape(M1 * M0, K1 * K0)[rows - 40:rows].cpu().numpy().astype(np.int64)
    b = rhs.permute(0, 2, 1, 3).reshape(N1 * N0, K1 * K0)[:cols].cpu().numpy().astype(np.int64)
    ref = a @ b.T + (init[rows - 40:].cpu().numpy() if accumulate else 0)
    assert np.array_equal(got[rows - 40:].cpu().numpy(), ref.astype(np.int32))


# The persistent kernels (one workgroup walks several output blocks with its
# software pipeline running across block boundaries). Forced, with the number
# of workgroups capped so that every workgroup owns several blocks even on
# these small problems: block counts that divide evenly over the workgroups
# and ones that do not, K of 8 steps (the minimum) and more, ACCUMULATE on and
# off (the case grid), tiles of 16 and 32 rows. Shapes are tile counts for
# (M0, N0, K0) so that rows/columns are whole 128x512 and 256x256 blocks.
@pytest.mark.parametrize("variant", [9, 10])
@pytest.mark.parametrize("tile", [(uk.MMT4D_TYPE_S8S8S32, 16, 16, 16, (512, 1024, 512)),
                                  (uk.MMT4D_TYPE_S8S8S32, 16, 16, 64, (512, 1536, 768)),
                                  (uk.MMT4D_TYPE_S8S8S32, 32, 8, 32, (256, 2560, 1024)),
                                  (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16, (512, 1024, 256)),
                                  (uk.MMT4D_TYPE_BF16BF16F32, 16, 32, 8, (512, 1536, 384)),
                                  (uk.MMT4D_TYPE_F32F32F32, 16, 16, 4, (256, 1024, 192))])
@pytest.mark.parametrize("workgroups", [1, 3, 4])
def test_mmt4d_persistent_kernels(gpu, oracle, variant, tile, workgroups):
    lib, torch = gpu
    tf, M0, N0, K0, (m, n, k) = tile
    lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant)
    lib.set_persistent_workgroups(workgroups)
    try:
        shape = (m // M0, n // N0, k // K0)
        for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=9100 + variant, slack=16,
                                             shapes=(shape,))):
            rng = np.random.default_rng(300 + ci)
            lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
            want = out0.copy()
            G.run_mmt4d_case(oracle, c, lhs, rhs, want)
            got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
            assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
            assert lib.last_kernel_name().endswith("_persistent"), lib.last_kernel_name()
    finally:
        lib.set_persistent_workgroups(0)
        lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)


def test_mmt4d_last_partial_round_runs_as_its_own_launch(gpu):
    """A problem that the 128x512 shape (and the 256x256 one) tiles exactly into
    1.25 rounds of blocks (320 on 256 compute units) is split by columns: whole
    rounds in one launch, the last 32 block columns in another with a smaller
    shape. Results equal the single launch of a forced shape bit for bit, the
    column scales of the dequantizing store included."""
    lib, torch = gpu
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S8S8S32, 16, 16, 16
    M1, N1, K1 = 256 // M0, 160 * 512 // N0, 512 // K0
    M, N = M1 * M0, N1 * N0
    g = torch.Generator(device="cuda"); g.manual_seed(33)
    lhs = torch.randint(-128, 128, (M1 * K1 * M0 * K0,), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1 * K1 * N0 * K0,), generator=g, device="cuda", dtype=torch.int8)
    acc0 = torch.randint(-1000, 1000, (M1 * N1 * M0 * N0,), generator=g, device="cuda", dtype=torch.int32)
    rs = torch.rand(M, generator=g, device="cuda") + 0.5
    cs = torch.rand(N, generator=g, device="cuda") + 0.5
    results = {}
    for mode in (uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_MFMA_VARIANT + 1):
        out = acc0.clone()
        y = torch.zeros(M, N, device="cuda", dtype=torch.float32)
        torch.cuda.synchronize()
        lib.set_kernel_mode(mode)
        try:
            lib.timing_begin()
            lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
                      N1 * M0 * N0, M1, N1, K1, M0, N0, K0, tf | uk.MMT4D_ACCUMULATE)
            launches = len(lib.timing_end())
            assert launches == (2 if mode == uk.KERNEL_MODE_AUTO else 1), launches
            name = lib.last_kernel_name()
            lib.mmt4d_dequant_unpack(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0,
                                     None, 0, 0, y.data_ptr(), 0, N, M, N, rs.data_ptr(), cs.data_ptr(),
                                     M1, N1, K1, M0, N0, K0, tf)
            lib.synchronize()
        finally:
            lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        results[mode] = (out.cpu(), y.cpu(), name)
    auto, forced = results[uk.KERNEL_MODE_AUTO], results[uk.KERNEL_MODE_MFMA_VARIANT + 1]
    assert auto[2] == "mmt4d_mfma_256x256_lds_direct" and forced[2] == "mmt4d_mfma_256x256_rhs_direct"
    assert torch.equal(auto[0], forced[0])
    assert torch.equal(auto[1], forced[1])
    # and against the integer product on a few rows and columns of both parts
    a = lhs.view(M1, K1, M0, K0).permute(0, 2, 1, 3).reshape(M, K1 * K0)[:32].cpu().to(torch.int64)
    for c0 in (0, 128 * 512 - 64, 128 * 512, N - 64):
        b = rhs.view(N1, K1, N0, K0).permute(0, 2, 1, 3).reshape(N, K1 * K0)[c0:c0 + 64].cpu().to(torch.int64)
        want = (a @ b.T).to(torch.int32)
        got = auto[0].view(M1, N1, M0, N0).permute(0, 2, 1, 3).reshape(M, N)[:32, c0:c0 + 64]
        base = acc0.view(M1, N1, M0, N0).permute(0, 2, 1, 3).reshape(M, N)[:32, c0:c0 + 64].cpu()
        assert torch.equal(got, want + base), c0


# Operands at odd element offsets and strides (the reference grid's slack of
# one element: tools/mmt4d_test.c:354-404), WITHOUT the generic-fallback flag:
# iree_uk_mmt4d_info advertises these tile shapes, so an MFMA kernel has to
# serve them wherever the buffers happen to start.
@pytest.mark.parametrize("variant", [0, 1, 3, 4])
@pytest.mark.parametrize("tile", [(uk.MMT4D_TYPE_S8S8S32, 16, 16, 2), (uk.MMT4D_TYPE_S8S8S32, 16, 16, 16),
                                  (uk.MMT4D_TYPE_S8S8S32, 32, 16, 8), (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16),
                                  (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 2),
                                  (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 32),
                                  (uk.MMT4D_TYPE_F32F32F32, 16, 16, 4)])
def test_mmt4d_unaligned_operands_take_the_mfma_kernels(gpu, oracle, tile, variant):
    lib, torch = gpu
    tf, M0, N0, K0 = tile
    lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
    before = lib.mfma_decline_count()
    bits = uk.MMT4D_TYPE_BITS[tf][0]
    kb = K0 * bits // 8
    shapes = ((1, 1, max(1, 64 // kb)), (3, 5, max(2, 200 // kb)), (17, 18, max(1, 128 // kb)),
              (1, 40, max(1, 512 // kb)), (2, 2, 3))
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=5200 + variant, slack=1, shapes=shapes)):
        rng = np.random.default_rng(700 + ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        assert lib.last_kernel_name().startswith("mmt4d_mfma"), (c.label(), lib.last_kernel_name())
    assert lib.mfma_decline_count() == before


def test_mmt4d_declined_call_is_counted_and_still_exact(gpu):
    """A negative panel stride is outside what the MFMA kernels index; without
    the fallback flag the call is still served (scalar kernel, same result)
    and shows in iree_uk_amd_mfma_decline_count."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, K1, M0, N0, K0 = 3, 2, 4, 16, 16, 16
    panel = K1 * M0 * K0
    g = torch.Generator(device="cuda"); g.manual_seed(77)
    lhs = torch.randint(-128, 128, (M1, panel), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1, K1 * N0 * K0), generator=g, device="cuda", dtype=torch.int8)
    fwd = torch.zeros(M1, N1 * M0 * N0, device="cuda", dtype=torch.int32)
    bwd = torch.zeros_like(fwd)
    before = lib.mfma_decline_count()
    lib.mmt4d(lhs.data_ptr(), 0, panel, rhs.data_ptr(), 0, K1 * N0 * K0, fwd.data_ptr(), 0,
              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32)
    assert lib.mfma_decline_count() == before
    lib.mmt4d(lhs.data_ptr(), (M1 - 1) * panel, -panel, rhs.data_ptr(), 0, K1 * N0 * K0,
              bwd.data_ptr(), 0, N1 * M0 * N0, M1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_generic"
    assert lib.mfma_decline_count() == before + 1
    assert torch.equal(bwd, fwd.flip(0))
