"""iree_uk_amd_mmt4d_dequant_unpack: mmt4d into a row-major f32 matrix with
per-row and per-column scales. The reference has no such call; what it must
equal is the composition its own pieces define: iree_uk_mmt4d into the tiled
accumulator buffer (mmt4d.c:55-114), iree_uk_unpack without transposes
(tools/unpack_test.c:13-58), then `(float)acc * row_scale[i] * col_scale[j]`
in f32, left to right. The oracle computes the first two; numpy's f32 multiply
and int32 -> f32 conversion (round to nearest even) the third."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk


def _want(oracle, c, lhs, rhs, acc_tiled, rows, cols, rs, cs, ok):
    """The composition on the CPU: returns the rows x cols f32 matrix."""
    M1, N1, M0, N0 = c.M, c.N, c.M0, c.N0
    tiled = acc_tiled.copy() if acc_tiled is not None else np.zeros(M1 * N1 * M0 * N0, np.int32)
    if c.K > 0 or not (c.flags & uk.MMT4D_ACCUMULATE):
        G.run_mmt4d_case(oracle, c, lhs, rhs, tiled.view(np.uint8))
    mat = np.zeros(rows * cols, np.int32)
    oracle.unpack(tiled, 0, N1 * M0 * N0, M0 * N0, mat, 0, cols, 1, M1, N1, M0, N0, rows, cols,
                  uk.UNPACK_TYPE_I32I32)
    mat = mat.reshape(rows, cols)
    v = mat.astype(np.float32) if ok == "s32" else mat.view(np.float32).copy()
    v = v * (rs[:, None] if rs is not None else np.float32(1))
    v = v * (cs[None, :] if cs is not None else np.float32(1))
    return v.astype(np.float32)


MODES = [uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_GENERIC, uk.KERNEL_MODE_MFMA_VARIANT + 1,
         uk.KERNEL_MODE_MFMA_VARIANT + 4, uk.KERNEL_MODE_MFMA_VARIANT + 5,
         uk.KERNEL_MODE_MFMA_VARIANT + 8, uk.KERNEL_MODE_MFMA_VARIANT + 16]


@pytest.mark.gpu
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("tf,M0,N0,K0", [
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 16), (uk.MMT4D_TYPE_S8S8S32, 32, 16, 8),
    (uk.MMT4D_TYPE_S8S8S32, 16, 16, 2), (uk.MMT4D_TYPE_S8S8S32, 8, 6, 4),
    (uk.MMT4D_TYPE_F16F16F32, 16, 16, 8), (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 8),
    (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 32), (uk.MMT4D_TYPE_F32F32F32, 16, 16, 1),
    (uk.MMT4D_TYPE_S16S16S32, 4, 6, 3), (uk.MMT4D_TYPE_S16S16S32, 16, 16, 2),
    (uk.MMT4D_TYPE_S16U4S32, 1, 32, 8), (uk.MMT4D_TYPE_S16S8S32, 8, 6, 4),
    (uk.MMT4D_TYPE_S8S4S32, 4, 8, 4),
    (uk.MMT4D_TYPE_S8S4S32, 16, 16, 16)])
def test_dequant_unpack_equals_mmt4d_unpack_scale(gpu, oracle, tf, M0, N0, K0, mode):
    """Bit for bit on the reference tests' small-integer inputs (every f32
    partial sum exact, so float types are order-independent too): ragged
    sizes, loose row pitch, an offset, ACCUMULATE from a strided tiled buffer,
    each scale present or absent, bytes outside the matrix untouched, device
    and host (staged) pointers."""
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    lk, rk, ok = T.MMT4D_KINDS[tf]
    k_whole = max(1, 3 * 128 * 8 // (K0 * uk.MMT4D_TYPE_BITS[tf][0]))  # whole 64/128-byte K steps
    shapes = [(3, 2, 5, 0, 0), (17, 18, 9, 5, 3), (1, 1, 1, 0, 15), (1, 40, 33, 15, 0),
              (2, 5, k_whole, 3, 2), (21, 1, k_whole, 0, 7), (5, 6, k_whole, 3, 2)]
    for si, (M1, N1, K1, cut0, cut1) in enumerate(shapes):
        for acc in (0, 1):
            rows, cols = M1 * M0 - min(cut0, M0 - 1), N1 * N0 - min(cut1, N0 - 1)
            pitch, off = cols + 3 * (si % 2), 5 * ((si + acc) % 2)
            acc_stride, acc_off = N1 * M0 * N0 + 8 * (si % 2), 4 * (si % 3)
            c = T.Mmt4dCase(tf | 0x200 | (uk.MMT4D_ACCUMULATE if acc else 0), M1, N1, K1, M0, N0,
                            K0, K1 * M0 * K0, K1 * N0 * K0, N1 * M0 * N0, 0, 0, 0)
            rng = np.random.default_rng(1000 * si + acc)
            lhs, rhs, _ = T.make_mmt4d_buffers(c, rng)
            acc_buf = rng.integers(-9, 9, acc_off + M1 * acc_stride).astype(np.int32)
            if ok != "s32":
                acc_buf = acc_buf.astype(np.float32).view(np.int32)
            acc_dense = np.concatenate([acc_buf[acc_off + i * acc_stride:][:N1 * M0 * N0]
                                        for i in range(M1)])
            rs = (rng.random(rows, dtype=np.float32) * 0.02 + 0.001) if (si + acc) % 3 != 1 else None
            cs = (rng.random(cols, dtype=np.float32) * 0.02 + 0.001) if si % 3 != 2 else None
            want_mat = _want(oracle, c, lhs, rhs, acc_dense if acc else None, rows, cols, rs, cs, ok)
            out0 = rng.random(off + rows * pitch, dtype=np.float32)
            want = out0.copy()
            for i in range(rows):
                want[off + i * pitch:off + i * pitch + cols] = want_mat[i]
            d = [T.DeviceBytes(torch, x) for x in (lhs, rhs, acc_buf, out0)]
            d_rs = T.DeviceBytes(torch, rs) if rs is not None else None
            d_cs = T.DeviceBytes(torch, cs) if cs is not None else None
            lib.mmt4d_dequant_unpack(
                d[0].ptr, 0, c.lhs_stride0, d[1].ptr, 0, c.rhs_stride0,
                d[2].ptr if acc else None, acc_off, acc_stride, d[3].ptr, off, pitch, rows, cols,
                d_rs.ptr if d_rs else None, d_cs.ptr if d_cs else None,
                M1, N1, K1, M0, N0, K0, c.flags)
            lib.synchronize()
            got = d[3].numpy().view(np.float32)
            assert np.array_equal(got.view(np.int32), want.view(np.int32)), (
                tf, M0, N0, K0, M1, N1, K1, acc, lib.last_kernel_name())
            assert np.array_equal(d[2].numpy().view(np.int32), acc_buf)   # accumulators only read
            host = out0.copy()
            lib.mmt4d_dequant_unpack(
                lhs.ctypes.data, 0, c.lhs_stride0, rhs.ctypes.data, 0, c.rhs_stride0,
                acc_buf.ctypes.data if acc else None, acc_off, acc_stride, host.ctypes.data, off,
                pitch, rows, cols, rs.ctypes.data if rs is not None else None,
                cs.ctypes.data if cs is not None else None, M1, N1, K1, M0, N0, K0, c.flags)
            assert np.array_equal(host.view(np.int32), want.view(np.int32))


@pytest.mark.gpu
def test_dequant_unpack_k_zero_still_scales_the_accumulators(gpu):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, M0, N0, K0 = 2, 3, 16, 16, 16
    rows, cols = 30, 41
    g = torch.Generator(device="cuda"); g.manual_seed(3)
    acc = torch.randint(-5000, 5000, (M1, N1, M0, N0), generator=g, device="cuda", dtype=torch.int32)
    rs = torch.rand(rows, generator=g, device="cuda") + 0.5
    cs = torch.rand(cols, generator=g, device="cuda") + 0.5
    dummy = torch.zeros(16, device="cuda", dtype=torch.int8)
    for accumulate in (0, 1):
        out = torch.full((rows, cols), -1.0, device="cuda")
        lib.mmt4d_dequant_unpack(dummy.data_ptr(), 0, 0, dummy.data_ptr(), 0, 0, acc.data_ptr(), 0,
                                 N1 * M0 * N0, out.data_ptr(), 0, cols, rows, cols, rs.data_ptr(),
                                 cs.data_ptr(), M1, N1, 0, M0, N0, K0,
                                 uk.MMT4D_TYPE_S8S8S32 | 0x200 | (uk.MMT4D_ACCUMULATE if accumulate else 0))
        lib.synchronize()
        mat = acc.permute(0, 2, 1, 3).reshape(M1 * M0, N1 * N0)[:rows, :cols]
        want = (mat.float() * rs[:, None]) * cs[None, :] if accumulate else torch.zeros_like(out)
        assert torch.equal(out, want)


@pytest.mark.gpu
@pytest.mark.parametrize("accumulate", [0, 1])
def test_dequant_unpack_with_remainder_strips(gpu, accumulate):
    """Large enough for the 256x256 variant, ragged against it in M and N (so
    strips are split off and take their share of the scales and accumulators)
    and with a K remainder (so the scales are applied by the second launch
    only): equal to mmt4d + unpack on the GPU, both pinned against the oracle
    elsewhere, followed by the two f32 multiplies."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, K1, M0, N0, K0 = 241, 273, 5, 16, 16, 16
    rows, cols = M1 * M0 - 3, N1 * N0 - 5
    g = torch.Generator(device="cuda"); g.manual_seed(11)
    lhs = torch.randint(-128, 128, (M1, K1, M0, K0), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1, K1, N0, K0), generator=g, device="cuda", dtype=torch.int8)
    acc = torch.randint(-10 ** 6, 10 ** 6, (M1 * N1 * M0 * N0,), generator=g, device="cuda",
                        dtype=torch.int32)
    rs = torch.rand(rows, generator=g, device="cuda") * 0.02 + 0.001
    cs = torch.rand(cols, generator=g, device="cuda") * 0.02 + 0.001
    flags = uk.MMT4D_TYPE_S8S8S32 | (uk.MMT4D_ACCUMULATE if accumulate else 0)
    tiled = acc.clone()
    lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, tiled.data_ptr(), 0,
              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags)
    mat = torch.zeros(rows, cols, device="cuda", dtype=torch.int32)
    lib.unpack(tiled.data_ptr(), 0, N1 * M0 * N0, M0 * N0, mat.data_ptr(), 0, cols, 1, M1, N1, M0, N0,
               rows, cols, uk.UNPACK_TYPE_I32I32)
    lib.synchronize()
    want = (mat.float() * rs[:, None]) * cs[None, :]
    got = torch.full((rows, cols), -1.0, device="cuda")
    lib.mmt4d_dequant_unpack(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0,
                             acc.data_ptr(), 0, N1 * M0 * N0, got.data_ptr(), 0, cols, rows, cols,
                             rs.data_ptr(), cs.data_ptr(), M1, N1, K1, M0, N0, K0, flags)
    assert lib.last_kernel_name().startswith(("mmt4d_mfma_256x256", "mmt4d_mfma_128x512"))
    lib.synchronize()
    assert torch.equal(got, want)


@pytest.mark.gpu
def test_decode_layer_fused_equals_the_integer_product_scaled(gpu):
    """The bench's decode-shaped layer (16 rows padded to M0 = 32, K = 4096,
    N = 14336, tiles 32x16x8, ACCUMULATE) through the fused call against the
    closed form: exact integer matmul of the unpacked operands plus the seeded
    accumulators, converted and scaled in f32."""
    lib, torch = gpu
    from iree_amd.runner import Runner
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    r = Runner(seed=0)   # takes over the library's stream and pointer mode
    try:
        wl = r.workload("c3_s8_decode_fused")
        k = wl.keep
        with torch.cuda.stream(r.stream):
            wl.ops[0].launch()
        r.stream.synchronize()
        assert lib.last_kernel_name() == "mmt4d_mfma_thin"
    finally:
        r.close()
    Mlog, N = k["act"].shape[0], k["w"].shape[0]
    prod = k["act"].cpu().to(torch.int64) @ k["w"].cpu().to(torch.int64).T          # [16][N]
    acc0 = k["out4"].view(k["N1"], k["M0"], k["N0"])[:, :Mlog, :].permute(1, 0, 2).reshape(Mlog, N)
    total = (prod + acc0.cpu().to(torch.int64)).to(torch.int32)
    want = (total.float() * k["scale_m"].cpu()[:, None]) * k["scale_n"].cpu()[None, :]
    assert torch.equal(k["y_fused"].cpu(), want)


def test_dequant_unpack_contract(lib):
    """Needs no device: a 16-bit out type, a matrix larger than the tiles and a
    missing accumulator buffer are contract violations; empty shapes return."""
    lib.raise_on_violation(True)   # (the session's setting; left on)
    def call(flags, rows=16, cols=16, acc=None, M=1):
        lib.mmt4d_dequant_unpack(None, 0, 0, None, 0, 0, acc, 0, 0, None, 0, cols, rows, cols,
                                 None, None, M, 1, 1, 16, 16, 16, flags)
    with pytest.raises(uk.ContractViolation):
        call(uk.MMT4D_TYPE_F16F16F16 | uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS)
    with pytest.raises(uk.ContractViolation):
        call(uk.MMT4D_TYPE_S8S8S32, rows=17)
    with pytest.raises(uk.ContractViolation):
        call(uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE)
    call(uk.MMT4D_TYPE_S8S8S32, rows=0)
    call(uk.MMT4D_TYPE_S8S8S32, rows=0, M=0)


@pytest.mark.gpu
def test_decode_without_pack_row_major_activations_are_m0_1_tiles(gpu):
    """A row-major [M, K] activation matrix is the mmt4d LHS layout with
    M0 = 1, so a decode step needs neither pack nor unpack on the activation
    side: mmt4d_dequant_unpack on M0 = 1 tiles against the exact product."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M, N, K, N0, K0 = 16, 2048, 4096, 16, 16
    g = torch.Generator(device="cuda"); g.manual_seed(9)
    act = torch.randint(-128, 128, (M, K), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (N, K), generator=g, device="cuda", dtype=torch.int8)
    rs = torch.rand(M, generator=g, device="cuda") * 0.02 + 0.001
    cs = torch.rand(N, generator=g, device="cuda") * 0.02 + 0.001
    N1, K1 = N // N0, K // K0
    rhs4 = torch.empty(N1 * K1 * N0 * K0, device="cuda", dtype=torch.int8)
    lib.pack(w.data_ptr(), 0, K, 1, rhs4.data_ptr(), 0, K1 * N0 * K0, N0 * K0, N, K, N1, K1, N0, K0, 0,
             uk.PACK_TYPE_I8I8)                       # weights: packed once
    y = torch.empty(M, N, device="cuda")
    lib.mmt4d_dequant_unpack(act.data_ptr(), 0, K, rhs4.data_ptr(), 0, K1 * N0 * K0, None, 0, 0,
                             y.data_ptr(), 0, N, M, N, rs.data_ptr(), cs.data_ptr(),
                             M, N1, K1, 1, N0, K0, uk.MMT4D_TYPE_S8S8S32)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_mfma_thin"
    prod = (act.cpu().to(torch.int64) @ w.cpu().to(torch.int64).T).to(torch.int32)
    want = (prod.float() * rs.cpu()[:, None]) * cs.cpu()[None, :]
    assert torch.equal(y.cpu(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("tf,M0,N0,K0,M1,N1,K1,name", [
    (uk.MMT4D_TYPE_S8S4S32, 16, 16, 16, 33, 9, 12, "mmt4d_mfma_s8s4_expanded"),
    (uk.MMT4D_TYPE_S16S8S32, 16, 16, 2, 9, 10, 64, "mmt4d_mfma_128x128_s16_widened"),
    (uk.MMT4D_TYPE_S16U4S32, 1, 32, 8, 130, 5, 16, "mmt4d_mfma_128x128_s16_widened"),
    (uk.MMT4D_TYPE_S8S8S32, 8, 8, 1, 33, 33, 272, "mmt4d_mfma_retiled")])
def test_dequant_unpack_on_operands_the_library_prepares_first(gpu, oracle, tf, M0, N0, K0, M1, N1, K1, name):
    """The calls whose operands the library widens or regroups before the
    matrix-core kernels run (4-bit weights from 512 rows on, s16 x s8 / u4 from
    128 rows and columns on, one-byte tile rows) through the fused entry point:
    ragged row-major result, ACCUMULATE from the tiled buffer, both scales."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lk, rk, ok = T.MMT4D_KINDS[tf]
    for acc in (0, 1):
        rows, cols = M1 * M0 - min(3, M0 - 1), N1 * N0 - min(5, N0 - 1)
        pitch, off = cols + 3, 5 * acc
        acc_stride, acc_off = N1 * M0 * N0 + 8, 4
        c = T.Mmt4dCase(tf | 0x200 | (uk.MMT4D_ACCUMULATE if acc else 0), M1, N1, K1, M0, N0,
                        K0, K1 * M0 * K0, K1 * N0 * K0, N1 * M0 * N0, 0, 0, 0)
        rng = np.random.default_rng(77 + acc)
        lhs, rhs, _ = T.make_mmt4d_buffers(c, rng)
        acc_buf = rng.integers(-9, 9, acc_off + M1 * acc_stride).astype(np.int32)
        acc_dense = np.concatenate([acc_buf[acc_off + i * acc_stride:][:N1 * M0 * N0] for i in range(M1)])
        rs = rng.random(rows, dtype=np.float32) * 0.02 + 0.001
        cs = rng.random(cols, dtype=np.float32) * 0.02 + 0.001
        want_mat = _want(oracle, c, lhs, rhs, acc_dense if acc else None, rows, cols, rs, cs, ok)
        out0 = rng.random(off + rows * pitch, dtype=np.float32)
        want = out0.copy()
        for i in range(rows):
            want[off + i * pitch:off + i * pitch + cols] = want_mat[i]
        d = [T.DeviceBytes(torch, x) for x in (lhs, rhs, acc_buf, out0, rs, cs)]
        lib.mmt4d_dequant_unpack(
            d[0].ptr, 0, c.lhs_stride0, d[1].ptr, 0, c.rhs_stride0,
            d[2].ptr if acc else None, acc_off, acc_stride, d[3].ptr, off, pitch, rows, cols,
            d[4].ptr, d[5].ptr, M1, N1, K1, M0, N0, K0, c.flags)
        lib.synchronize()
        assert lib.last_kernel_name() == name, lib.last_kernel_name()
        got = d[3].numpy().view(np.float32)
        assert np.array_equal(got.view(np.int32), want.view(np.int32)), (tf, acc)
