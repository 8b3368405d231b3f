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
