"""Oracle (our C restatement) against the compiled reference C ukernels, buffer
for buffer, on the seeded sweep shaped like the reference's own unit tests.
Skipped where oracle/_ref was not built (its digests are still checked by
test_oracle_golden.py). Runs without a GPU."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk


@pytest.mark.parametrize("n", range(len(G.PACK_TILES)))
def test_pack_sweep(oracle, reference, n):
    tf, t0, t1 = G.PACK_TILES[n]
    for ci, c in enumerate(T.pack_cases(tf, t0, t1, seed=7000 + n)):
        rng = np.random.default_rng(ci)
        inp, out0 = T.make_pack_buffers(c, rng)
        a, b = out0.copy(), out0.copy()
        G.run_pack_case(oracle, c, inp, a)
        G.run_pack_case(reference, c, inp, b)
        assert np.array_equal(a, b), c.label()


@pytest.mark.parametrize("n", range(len(G.UNPACK_TILES)))
def test_unpack_sweep(oracle, reference, n):
    tf, t0, t1 = G.UNPACK_TILES[n]
    for ci, c in enumerate(T.unpack_cases(tf, t0, t1, seed=8000 + n)):
        rng = np.random.default_rng(ci)
        inp, out0 = T.make_unpack_buffers(c, rng)
        a, b = out0.copy(), out0.copy()
        G.run_unpack_case(oracle, c, inp, a)
        G.run_unpack_case(reference, c, inp, b)
        assert np.array_equal(a, b), c.label()


@pytest.mark.parametrize("n", range(len(G.MMT4D_TILES)))
def test_mmt4d_sweep(oracle, reference, n):
    tf, M0, N0, K0, extra = G.MMT4D_TILES[n]
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=9000 + n, extra_flags=extra)):
        rng = np.random.default_rng(ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        a, b = out0.copy(), out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, a)
        G.run_mmt4d_case(reference, c, lhs, rhs, b)
        assert np.array_equal(a, b), c.label()


def test_mmt4d_random_normal_floats_bit_identical(oracle, reference):
    """Beyond small integers: on N(0,1) f16/bf16 inputs the oracle reproduces
    the reference's generic path bit for bit (same order, separate multiply and
    add, same subnormal flush)."""
    rng = np.random.default_rng(3)
    for tf, conv in ((uk.MMT4D_TYPE_F16F16F32, lambda v: v.astype(np.float16).view(np.uint16)),
                     (uk.MMT4D_TYPE_BF16BF16F32, T.f32_to_bf16_bits)):
        M, N, K, M0, N0, K0 = 3, 2, 17, 16, 16, 16
        lhs = conv(rng.standard_normal(M * K * M0 * K0).astype(np.float32) * 1e-3)
        rhs = conv(rng.standard_normal(N * K * N0 * K0).astype(np.float32))
        a = np.zeros(M * N * M0 * N0, dtype=np.float32)
        b = a.copy()
        args = (0, K * M0 * K0, rhs, 0, K * N0 * K0)
        oracle.mmt4d(lhs, *args, a, 0, N * M0 * N0, M, N, K, M0, N0, K0, tf | 0x200)
        reference.mmt4d(lhs, *args, b, 0, N * M0 * N0, M, N, K, M0, N0, K0, tf | 0x200)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_reference_arch_paths_agree_on_integers(oracle, reference):
    """The reference's AVX-512(-VNNI) s8 tile functions give the same bytes as
    its generic path, hence as the oracle: what the CPU baseline times is the
    same function."""
    from oracle import uk_oracle
    ref_arch = uk_oracle.Checker("reference").use_host_cpu_features(True)
    if not int(ref_arch.cpu_data[0]):
        pytest.skip("host reports no x86-64 SIMD features")
    rng = np.random.default_rng(4)
    M, N, K, M0, N0, K0 = 5, 7, 33, 16, 16, 2
    lhs = rng.integers(-128, 128, M * K * M0 * K0).astype(np.int8)
    rhs = rng.integers(-128, 128, N * K * N0 * K0).astype(np.int8)
    a = rng.integers(-1000, 1000, M * N * M0 * N0).astype(np.int32)
    b = a.copy()
    oracle.mmt4d(lhs, 0, K * M0 * K0, rhs, 0, K * N0 * K0, a, 0, N * M0 * N0,
                 M, N, K, M0, N0, K0, 0x302)
    ref_arch.mmt4d(lhs, 0, K * M0 * K0, rhs, 0, K * N0 * K0, b, 0, N * M0 * N0,
                   M, N, K, M0, N0, K0, 0x102)  # no generic fallback allowed
    assert np.array_equal(a, b)


def _ref_f8(reference):
    import ctypes
    L = reference.lib
    if not hasattr(L, "ref_f8e4m3fn_to_f32"):
        pytest.skip("oracle/_ref was built without the f8 conversions")
    L.ref_f8e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
    L.ref_f8e4m3fn_to_f32.restype = ctypes.c_float
    L.ref_f32_to_f8e4m3fn.argtypes = [ctypes.c_float]
    L.ref_f32_to_f8e4m3fn.restype = ctypes.c_uint8
    return L


def test_f8_decode_all_codes_against_reference_code(oracle, reference):
    """The oracle's E4M3FN decode (what its f8 mmt4d multiplies) against the
    reference's own iree_math_f8e4m3fn_to_f32
    (runtime/src/iree/base/internal/math.h:324-362,557-560), compiled from
    where it lies: all 256 codes bit for bit, NaNs as NaNs."""
    L = _ref_f8(reference)
    for v in range(256):
        want = np.float32(L.ref_f8e4m3fn_to_f32(v))
        got = np.float32(oracle.f8e4m3fn_to_f32(v))
        if np.isnan(want):
            assert np.isnan(got), hex(v)
        else:
            assert got.view(np.uint32) == want.view(np.uint32), hex(v)
    assert sum(np.float64(L.ref_f8e4m3fn_to_f32(v)) for v in range(0x7F)) == 5407.875


def test_f8_test_side_encoder_against_reference_encoder(reference):
    """The encoder the tests use to make f8 inputs against the reference's
    iree_math_f32_to_f8e4m3fn (math.h:364-460) on every representable value,
    on midpoints between neighbours (ties to even) and on random values in
    range. One known difference is left out: the reference flushes magnitudes
    inside (2^-10, 2^-9) to zero instead of rounding them up to the minimum
    subnormal (math.h:431-442)."""
    L = _ref_f8(reference)
    table = T.f8e4m3fn_table()
    finite = [v for v in range(256) if not np.isnan(table[v])]
    vals = [float(table[v]) for v in finite]
    pos = sorted(set(abs(x) for x in vals))
    mids = [(a + b) / 2 for a, b in zip(pos[:-1], pos[1:])]
    rng = np.random.default_rng(11)
    rand = list(rng.uniform(-448, 448, 4000)) + list(rng.normal(0, 1, 4000))
    probe = np.array(vals + mids + [-m for m in mids] + rand, dtype=np.float32)
    tiny = (np.abs(probe) > 2.0 ** -10) & (np.abs(probe) < 2.0 ** -9)
    probe = probe[~tiny]
    ours = T.f32_to_f8e4m3fn_bits(probe)
    for x, code in zip(probe, ours):
        want = int(L.ref_f32_to_f8e4m3fn(float(x)))
        # +0 and -0 of a value that rounds to zero keep their sign in both
        assert int(code) == want, (float(x), hex(int(code)), hex(want))
