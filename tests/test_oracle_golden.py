"""Pins the CPU oracle (oracle/uk_oracle.c) against vectors that do not come
from the oracle itself: golden tensors held by the reference's own tests,
known-answer vectors produced by running the compiled reference, closed forms,
and numpy reshape/transpose identities. Runs without a GPU."""
import json
import os

import numpy as np
import pytest

import uk_testing as T
from iree_amd import ukernel as uk

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _pack_dense(chk, x, out_shape, flags, pad=0):
    """pack a dense 2-D array into a dense 4-D array of out_shape."""
    o0, o1, o2, o3 = out_shape
    out = np.zeros(out_shape, dtype=x.dtype)
    chk.pack(np.ascontiguousarray(x), 0, x.shape[1], 1, out, 0, o1 * o2 * o3,
             o2 * o3, x.shape[0], x.shape[1], o0, o1, o2, o3, pad, flags)
    return out


def _unpack_dense(chk, x4, out_shape, flags):
    i0, i1, i2, i3 = x4.shape
    out = np.zeros(out_shape, dtype=x4.dtype)
    chk.unpack(np.ascontiguousarray(x4), 0, i1 * i2 * i3, i2 * i3, out, 0,
               out_shape[1], 1, i0, i1, i2, i3, out_shape[0], out_shape[1], flags)
    return out


# ---- golden tensors of the reference's e2e tests --------------------------

def test_pack_mlir_static_golden(oracle):
    # tests/e2e/linalg/pack.mlir:21-27: 4x4 i32 iota, inner tiles [2,2].
    x = np.arange(16, dtype=np.int32).reshape(4, 4)
    got = _pack_dense(oracle, x, (2, 2, 2, 2), uk.PACK_TYPE_I32I32)
    want = [[[[0, 1], [4, 5]], [[2, 3], [6, 7]]],
            [[[8, 9], [12, 13]], [[10, 11], [14, 15]]]]
    assert got.tolist() == want


def test_pack_mlir_padding_golden(oracle):
    # tests/e2e/linalg/pack.mlir:51-68: 4x4 iota, tiles [3,3], padding 0.
    x = np.arange(16, dtype=np.int32).reshape(4, 4)
    got = _pack_dense(oracle, x, (2, 2, 3, 3), uk.PACK_TYPE_I32I32, pad=0)
    want = [[[[0, 1, 2], [4, 5, 6], [8, 9, 10]],
             [[3, 0, 0], [7, 0, 0], [11, 0, 0]]],
            [[[12, 13, 14], [0, 0, 0], [0, 0, 0]],
             [[15, 0, 0], [0, 0, 0], [0, 0, 0]]]]
    assert got.tolist() == want


def test_unpack_mlir_golden(oracle):
    # tests/e2e/linalg/unpack.mlir:24-31: inverse of the static pack above.
    x4 = np.array([[[[0, 1], [4, 5]], [[2, 3], [6, 7]]],
                   [[[8, 9], [12, 13]], [[10, 11], [14, 15]]]], dtype=np.int32)
    got = _unpack_dense(oracle, x4, (4, 4), uk.UNPACK_TYPE_I32I32)
    assert got.tolist() == np.arange(16).reshape(4, 4).tolist()


def test_unpack_mlir_extract_slice_golden(oracle):
    # tests/e2e/linalg/unpack.mlir:50-59: [2][2][3][3] -> 4x4, dropping padding.
    x4 = np.array([[[[0, 1, 2], [4, 5, 6], [8, 9, 10]],
                    [[3, 0, 0], [7, 0, 0], [11, 0, 0]]],
                   [[[12, 13, 14], [0, 0, 0], [0, 0, 0]],
                    [[15, 0, 0], [0, 0, 0], [0, 0, 0]]]], dtype=np.int32)
    got = _unpack_dense(oracle, x4, (4, 4), uk.UNPACK_TYPE_I32I32)
    assert got.tolist() == np.arange(16).reshape(4, 4).tolist()


# ---- known-answer vectors from the compiled reference ---------------------

def _kat():
    with open(os.path.join(GOLDEN, "reference_kat.json")) as f:
        return json.load(f)


def test_pack_kat(oracle):
    for case in _kat()["pack"]:
        x = np.array(case["in"], dtype=np.int8).reshape(3, 5)
        o0, o1 = case["out_size01"]
        out = np.full(o0 * o1 * 6, 99, dtype=np.int8)
        oracle.pack(x, 0, 5, 1, out, 0, o1 * 6, 6, 3, 5, o0, o1, 2, 3, 0xEE,
                    case["flags"])
        assert out.tolist() == case["out"], hex(case["flags"])


def test_unpack_kat(oracle):
    for case in _kat()["unpack"]:
        i0, i1 = case["in_size01"]
        x = np.arange(i0 * i1 * 6, dtype=np.int32)
        out = np.full(15, -1, dtype=np.int32)
        oracle.unpack(x, 0, i1 * 6, 6, out, 0, 5, 1, i0, i1, 2, 3, 3, 5,
                      case["flags"])
        assert out.tolist() == case["out"], hex(case["flags"])


def test_mmt4d_kat(oracle):
    for case in _kat()["mmt4d_s8"]:
        lhs = np.array(case["lhs"], dtype=np.int8)
        rhs = np.array(case["rhs"], dtype=np.int8)
        out = np.array(case["out_init"], dtype=np.int32)
        oracle.mmt4d(lhs, 0, 8, rhs, 0, 8, out, 0, 4, 1, 1, 2, 2, 2, 2, case["flags"])
        assert out.tolist() == case["out"]


def test_mmt4d_f16_subnormal_flush_kat(oracle):
    # The reference generic path flushes f16 subnormal inputs
    # (runtime/src/iree/builtins/ukernel/common.h:685-686): 2.0, not 2.0039.
    case = _kat()["mmt4d_f16_flush"]
    lhs = np.array(case["lhs"], dtype=np.uint16)
    rhs = np.array(case["rhs"], dtype=np.uint16)
    out = np.zeros(1, dtype=np.float32)
    oracle.mmt4d(lhs, 0, 2, rhs, 0, 2, out, 0, 1, 1, 1, 1, 1, 1, 2,
                 uk.MMT4D_TYPE_F16F16F32 | 0x200)
    assert out[0] == np.float32(case["out"])


def test_golden_sweep_fixture(oracle):
    """Outputs of the compiled reference on seeded inputs, stored as SHA-256
    digests by tests/golden/make_golden.py; the oracle must reproduce them."""
    import hashlib
    from golden import make_golden
    with open(os.path.join(GOLDEN, "reference_sweep.json")) as f:
        want = json.load(f)
    got = make_golden.sweep_digests(oracle)
    assert got.keys() == want.keys()
    bad = [k for k in want if want[k] != got[k]]
    assert not bad, bad[:5]


# ---- f8E4M3FN -------------------------------------------------------------

def test_f8_decode_closed_form(oracle):
    table = T.f8e4m3fn_table()
    for v in range(256):
        got = np.float32(oracle.f8e4m3fn_to_f32(v))
        if np.isnan(table[v]):
            assert np.isnan(got), v
        else:
            assert got == table[v] and np.signbit(got) == np.signbit(table[v]), v


def test_f8_decode_known_values(oracle):
    # runtime/src/iree/base/internal/math_test.cc:483-589 and further known-answer values.
    kv = {0x01: 2.0 ** -9, 0x07: 7 * 2.0 ** -9, 0x08: 2.0 ** -6,
          0x0F: 0.029296875, 0x28: 0.25, 0x38: 1.0, 0x40: 2.0, 0x77: 240.0,
          0x78: 256.0, 0x7E: 448.0, 0xB8: -1.0, 0xFE: -448.0, 0xED: -104.0}
    for code, val in kv.items():
        assert oracle.f8e4m3fn_to_f32(code) == val, hex(code)
    assert np.isnan(oracle.f8e4m3fn_to_f32(0x7F))
    assert np.isnan(oracle.f8e4m3fn_to_f32(0xFF))
    z = np.float32(oracle.f8e4m3fn_to_f32(0x80))
    assert z == 0 and np.signbit(z)
    s = sum(np.float64(oracle.f8e4m3fn_to_f32(v)) for v in range(0x7F))
    assert s == 5407.875
    s2 = sum(np.float64(oracle.f8e4m3fn_to_f32(v)) ** 2 for v in range(0x7F))
    assert abs(s2 - 1271466.665802002) < 1e-6


def test_f8_encoder_helper_matches_reference_kats():
    # The test-side encoder (not part of the product) against
    # math_test.cc:483-550 values that do not involve the reference's
    # flush of (2^-10, 2^-9).
    enc = T.f32_to_f8e4m3fn_bits
    for val, code in ((0.25, 0x28), (-100.375, 0xED), (448.0, 0x7E),
                      (0.3, 0x2A), (-1.7, 0xBE), (447.9, 0x7E), (1 / 512, 0x01)):
        assert int(enc(np.array([val], dtype=np.float32))[0]) == code, val


# ---- identities -----------------------------------------------------------

@pytest.mark.parametrize("ti", [False, True])
@pytest.mark.parametrize("to", [False, True])
@pytest.mark.parametrize("shape,tile", [((37, 53), (4, 8)), ((64, 48), (16, 16)),
                                        ((5, 7), (3, 2)), ((33, 1), (16, 1))])
def test_pack_equals_pad_reshape_transpose(oracle, shape, tile, ti, to):
    rng = np.random.default_rng(5)
    x = rng.integers(-1000, 1000, shape).astype(np.int32)
    want = T.numpy_pack(x, tile[0], tile[1], ti, to, pad=-7)
    flags = uk.PACK_TYPE_I32I32 | (0x100 if ti else 0) | (0x200 if to else 0)
    got = _pack_dense(oracle, x, want.shape, flags, pad=(-7) & 0xFFFFFFFFFFFFFFFF)
    assert np.array_equal(got, want)
    back = _unpack_dense(oracle, got, shape, flags)
    assert np.array_equal(back, x)


def test_pack_matmul_operand_forms(oracle):
    # tests/e2e/linalg/pack_i8.mlir:26-46: LHS [M,K] -> [M1][K1][M0][K0], no
    # flags; :48-68: row-major RHS [K,N] -> [N1][K1][N0][K0] is
    # reshape [K1,K0,N1,N0] + permute (2,0,3,1) = TRANSPOSE_INNER|OUTER.
    rng = np.random.default_rng(6)
    M, K, N, M0, N0, K0 = 32, 24, 48, 8, 16, 4
    lhs = rng.integers(-128, 128, (M, K)).astype(np.int8)
    rhs = rng.integers(-128, 128, (K, N)).astype(np.int8)
    want_l = lhs.reshape(M // M0, M0, K // K0, K0).transpose(0, 2, 1, 3)
    got_l = _pack_dense(oracle, lhs, want_l.shape, uk.PACK_TYPE_I8I8)
    assert np.array_equal(got_l, want_l)
    want_r = rhs.reshape(K // K0, K0, N // N0, N0).transpose(2, 0, 3, 1)
    got_r = _pack_dense(oracle, rhs, want_r.shape, uk.PACK_TYPE_I8I8 | 0x300)
    assert np.array_equal(got_r, want_r)


def test_padding_uses_low_bytes_only(oracle):
    x = np.zeros((1, 1), dtype=np.uint16)
    out = np.zeros((1, 1, 2, 2), dtype=np.uint16)
    oracle.pack(x, 0, 1, 1, out, 0, 4, 4, 1, 1, 1, 1, 2, 2, 0x1122334455667788,
                uk.PACK_TYPE_F16F16)
    assert out.ravel().tolist() == [0, 0x7788, 0x7788, 0x7788]


# ---- mmt4d against brute force --------------------------------------------

def _matmul_via_mmt4d(oracle, a, b_t, M0, N0, K0, type_flag, out_dtype, acc=None):
    """a: [M,K], b_t: [N,K] (storage dtype). Packs with numpy, runs the oracle
    mmt4d, unpacks with numpy; returns [M,N]."""
    M, K = a.shape
    N = b_t.shape[0]
    lhs4 = a.reshape(M // M0, M0, K // K0, K0).transpose(0, 2, 1, 3).copy()
    rhs4 = b_t.reshape(N // N0, N0, K // K0, K0).transpose(0, 2, 1, 3).copy()
    out4 = np.zeros((M // M0, N // N0, M0, N0), dtype=out_dtype)
    flags = type_flag | 0x200
    if acc is not None:
        out4[:] = acc.reshape(M // M0, M0, N // N0, N0).transpose(0, 2, 1, 3)
        flags |= uk.MMT4D_ACCUMULATE
    oracle.mmt4d(lhs4, 0, lhs4[0].size, rhs4, 0, rhs4[0].size, out4, 0,
                 out4[0].size, M // M0, N // N0, K // K0, M0, N0, K0, flags)
    return out4.transpose(0, 2, 1, 3).reshape(M, N)


def test_mmt4d_s8_equals_integer_matmul(oracle):
    rng = np.random.default_rng(7)
    a = rng.integers(-128, 128, (48, 40)).astype(np.int8)
    b = rng.integers(-128, 128, (36, 40)).astype(np.int8)
    want = a.astype(np.int64) @ b.astype(np.int64).T
    for (M0, N0, K0) in ((16, 12, 2), (8, 4, 8), (3, 9, 5), (48, 36, 40), (1, 1, 1)):
        got = _matmul_via_mmt4d(oracle, a, b, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32, np.int32)
        assert np.array_equal(got, want), (M0, N0, K0)
    acc = rng.integers(-2 ** 31, 2 ** 31, (48, 36)).astype(np.int32)
    got = _matmul_via_mmt4d(oracle, a, b, 16, 12, 2, uk.MMT4D_TYPE_S8S8S32, np.int32, acc)
    want_acc = ((want + acc.astype(np.int64) + 2 ** 31) % 2 ** 32 - 2 ** 31)
    assert np.array_equal(got, want_acc)  # wraps modulo 2^32


@pytest.mark.parametrize("type_flag,kind", [(uk.MMT4D_TYPE_F32F32F32, "f32"),
                                            (uk.MMT4D_TYPE_F16F16F32, "f16"),
                                            (uk.MMT4D_TYPE_BF16BF16F32, "bf16"),
                                            (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, "f8")])
def test_mmt4d_float_exact_on_small_integers(oracle, type_flag, kind):
    """With small-integer inputs every product and partial sum is exact in
    f32, so the result equals the integer matmul whatever the order."""
    rng = np.random.default_rng(8)
    M, N, K = 32, 24, 64
    ai = rng.integers(-4, 5, (M, K))
    bi = rng.integers(-4, 5, (N, K))
    enc = {"f32": lambda v: v.astype(np.float32),
           "f16": lambda v: v.astype(np.float16).view(np.uint16),
           "bf16": lambda v: T.f32_to_bf16_bits(v.astype(np.float32)),
           "f8": lambda v: T.f32_to_f8e4m3fn_bits(v.astype(np.float32))}[kind]
    got = _matmul_via_mmt4d(oracle, enc(ai), enc(bi), 8, 4, 16, type_flag, np.float32)
    assert np.array_equal(got, (ai @ bi.T).astype(np.float32))


def test_mmt4d_f16_sequential_f32_definition(oracle):
    """On random normal f16 inputs the result is the sequential f32 sum in
    (k, k0) order with a separate multiply and add."""
    rng = np.random.default_rng(9)
    M0, N0, K0, K = 2, 3, 4, 5
    lhs = rng.standard_normal((K, M0, K0)).astype(np.float16)
    rhs = rng.standard_normal((K, N0, K0)).astype(np.float16)
    out = np.zeros((M0, N0), dtype=np.float32)
    oracle.mmt4d(lhs.view(np.uint16), 0, lhs.size, rhs.view(np.uint16), 0,
                 rhs.size, out, 0, out.size, 1, 1, K, M0, N0, K0,
                 uk.MMT4D_TYPE_F16F16F32 | 0x200)
    for i in range(M0):
        for j in range(N0):
            acc = np.float32(0)
            for k in range(K):
                for k0 in range(K0):
                    p = np.float32(lhs[k, i, k0]) * np.float32(rhs[k, j, k0])
                    acc = np.float32(acc + p)
            assert out[i, j] == acc


def test_mmt4d_k0_and_accumulate_invariants(oracle):
    rng = np.random.default_rng(10)
    out0 = rng.integers(-100, 100, 2 * 3 * 4).astype(np.int32)
    lhs = np.zeros(1, np.int8)
    rhs = np.zeros(1, np.int8)
    out = out0.copy()
    # K == 0 with ACCUMULATE: untouched (mmt4d.c:106-114).
    oracle.mmt4d(lhs, 0, 0, rhs, 0, 0, out, 0, 12, 2, 1, 0, 3, 4, 2, 0x302)
    assert np.array_equal(out, out0)
    # K == 0 without ACCUMULATE: zero fill.
    oracle.mmt4d(lhs, 0, 0, rhs, 0, 0, out, 0, 12, 2, 1, 0, 3, 4, 2, 0x202)
    assert not out.any()
    # M == 0 / N == 0: untouched.
    out = out0.copy()
    oracle.mmt4d(lhs, 0, 0, rhs, 0, 0, out, 0, 12, 0, 1, 1, 3, 4, 2, 0x202)
    oracle.mmt4d(lhs, 0, 0, rhs, 0, 0, out, 0, 12, 2, 0, 1, 3, 4, 2, 0x202)
    assert np.array_equal(out, out0)
