"""Seeded random sweeps of pack / unpack / mmt4d on the GPU against the oracle,
through the C-ABI: shapes, tile sizes, strides, offsets and flags drawn at
random (mid-size, so that the streaming, tiled and generic kernels and several
MFMA variants are all reached), whole destination buffers compared bit for
bit. Complements the reference's own test grids with shapes they do not hold."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

PACK_TYPES = [uk.PACK_TYPE_F32F32, uk.PACK_TYPE_I8I8, uk.PACK_TYPE_I32I32, uk.PACK_TYPE_F16F16,
              uk.PACK_TYPE_BF16BF16]
UNPACK_TYPES = [uk.UNPACK_TYPE_F32F32, uk.UNPACK_TYPE_I32I32, uk.UNPACK_TYPE_F16F16,
                uk.UNPACK_TYPE_BF16BF16]
TILE_SIDES = [1, 2, 3, 4, 6, 8, 16, 32, 64]


def _pack_case(rng, tf):
    es = uk.PACK_TYPE_BYTES[tf]
    while True:
        t0, t1 = (int(rng.choice(TILE_SIDES)) for _ in range(2))
        if t0 * t1 * es <= 4096:
            break
    o0, o1 = int(rng.integers(1, 40)), int(rng.integers(1, 40))
    ti, to = int(rng.integers(0, 2)), int(rng.integers(0, 2))
    flags = tf | (uk.PACK_TRANSPOSE_INNER if ti else 0) | (uk.PACK_TRANSPOSE_OUTER if to else 0)
    lt0, lt1 = (t1, t0) if ti else (t0, t1)            # logical tile along matrix dims 0, 1
    lo0, lo1 = (o1, o0) if to else (o0, o1)            # logical outer counts
    in0 = max(0, lo0 * lt0 - int(rng.integers(0, lt0 + 3)))
    in1 = max(0, lo1 * lt1 - int(rng.integers(0, lt1 + 3)))
    in_stride1 = 1 if rng.integers(0, 4) else 2
    in_stride0 = in1 * in_stride1 + int(rng.choice([0, 0, 1, 4, 16]))
    out_stride0 = o1 * t0 * t1 + int(rng.choice([0, 0, 1, 4, 16]))
    return T.PackCase(flags, in0, in1, o0, o1, t0, t1, in_stride0, in_stride1, out_stride0,
                      int(rng.choice([0, 1, 4, 16])), int(rng.choice([0, 1, 4, 16])),
                      int(rng.integers(0, 2 ** 63)))


def _unpack_case(rng, tf):
    es = uk.PACK_TYPE_BYTES[tf]
    while True:
        t0, t1 = (int(rng.choice(TILE_SIDES)) for _ in range(2))
        if t0 * t1 * es <= 4096:
            break
    i0, i1 = int(rng.integers(1, 40)), int(rng.integers(1, 40))
    ti, to = int(rng.integers(0, 2)), int(rng.integers(0, 2))
    flags = tf | (uk.UNPACK_TRANSPOSE_INNER if ti else 0) | (uk.UNPACK_TRANSPOSE_OUTER if to else 0)
    lt0, lt1 = (t1, t0) if ti else (t0, t1)
    lo0, lo1 = (i1, i0) if to else (i0, i1)
    out0 = max(1, lo0 * lt0 - int(rng.integers(0, lt0)))
    out1 = max(1, lo1 * lt1 - int(rng.integers(0, lt1)))
    out_stride1 = 1 if rng.integers(0, 4) else 2
    out_stride0 = out1 * out_stride1 + int(rng.choice([0, 0, 1, 4, 16]))
    in_stride0 = i1 * t0 * t1 + int(rng.choice([0, 0, 1, 4, 16]))
    return T.UnpackCase(flags, i0, i1, t0, t1, out0, out1, in_stride0, out_stride0, out_stride1,
                        int(rng.choice([0, 1, 4, 16])), int(rng.choice([0, 1, 4, 16])))


def test_pack_random_sweep(gpu, oracle):
    lib, torch = gpu
    rng = np.random.default_rng(2024)
    kernels = set()
    for ci in range(160):
        c = _pack_case(rng, PACK_TYPES[ci % len(PACK_TYPES)])
        inp, out = T.make_pack_buffers(c, np.random.default_rng(ci))
        want = out.copy()
        G.run_pack_case(oracle, c, inp, want)
        got = T.gpu_pack(lib, torch, c, inp, out)
        assert np.array_equal(got, want), (ci, c, lib.last_kernel_name())
        kernels.add(lib.last_kernel_name())
    assert {"pack_stream", "pack_generic"} <= kernels, kernels


def test_pack_random_sweep_element_transpositions(gpu, oracle):
    """Every element size with TRANSPOSE_INNER, and untransposed tiles with rows
    of one, two or four bytes, at sizes of several 32-row x 512-byte blocks: the
    domain of the element-transposing kernel (most cases) and its borders (tile
    sides that are not powers of two, rows that are only 2-byte aligned, tiles
    too small for a 16-byte vector), which other kernels serve."""
    lib, torch = gpu
    rng = np.random.default_rng(77)
    served = 0
    for ci in range(200):
        tf = [uk.PACK_TYPE_I8I8, uk.PACK_TYPE_F16F16, uk.PACK_TYPE_BF16BF16, uk.PACK_TYPE_F32F32,
              uk.PACK_TYPE_I32I32][ci % 5]
        es = uk.PACK_TYPE_BYTES[tf]
        ti = int(rng.integers(0, 4)) != 0
        if ti:
            s2 = int(rng.choice([1, 2, 4, 8, 16, 32, 64, 12]))       # columns of the matrix per tile
            s3 = int(rng.choice([2, 4, 8, 16, 32, 64, 6]))           # rows of the matrix per tile
        else:
            s2, s3 = int(rng.choice([4, 8, 16, 32, 64, 24])), int(rng.choice([1, 2, 4][:3 - es // 2]))
        if s2 * s3 * es > 4096:
            continue
        a0, a1 = (s3, s2) if ti else (s2, s3)
        in0, in1 = int(rng.integers(1, 330)), int(rng.integers(1, 700))
        if not ti and s3 > 1 and rng.integers(0, 4):
            in1 = -(-in1 // s3) * s3
        to = int(rng.integers(0, 2))
        o0 = -(-in0 // a0) + int(rng.integers(0, 2))
        o1 = -(-in1 // a1) + int(rng.integers(0, 3))
        os0, os1 = (o1, o0) if to else (o0, o1)
        flags = tf | (uk.PACK_TRANSPOSE_INNER if ti else 0) | (uk.PACK_TRANSPOSE_OUTER if to else 0)
        align = 1 if rng.integers(0, 6) == 0 else 4
        in_stride0 = -(-(in1 + int(rng.integers(0, 9))) // align) * align
        c = T.PackCase(flags, in0, in1, os0, os1, s2, s3, in_stride0, 1,
                       os1 * s2 * s3 + int(rng.choice([0, 0, 16, 48])),
                       int(rng.choice([0, 4, 20])), int(rng.choice([0, 16, 32])), int(rng.integers(0, 2 ** 63)))
        inp, out = T.make_pack_buffers(c, np.random.default_rng(ci))
        want = out.copy()
        G.run_pack_case(oracle, c, inp, want)
        got = T.gpu_pack(lib, torch, c, inp, out)
        assert np.array_equal(got, want), (ci, c, lib.last_kernel_name())
        served += lib.last_kernel_name() == "pack_transposing"
    assert served >= 80, served


def test_unpack_random_sweep(gpu, oracle):
    lib, torch = gpu
    rng = np.random.default_rng(2025)
    kernels = set()
    for ci in range(160):
        c = _unpack_case(rng, UNPACK_TYPES[ci % len(UNPACK_TYPES)])
        inp, out = T.make_unpack_buffers(c, np.random.default_rng(ci))
        want = out.copy()
        G.run_unpack_case(oracle, c, inp, want)
        got = T.gpu_unpack(lib, torch, c, inp, out)
        assert np.array_equal(got, want), (ci, c, lib.last_kernel_name())
        kernels.add(lib.last_kernel_name())
    assert {"unpack_stream", "unpack_generic"} <= kernels, kernels


MMT4D_TYPES = [uk.MMT4D_TYPE_S8S8S32, uk.MMT4D_TYPE_F16F16F32, uk.MMT4D_TYPE_BF16BF16F32,
               uk.MMT4D_TYPE_F32F32F32, uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, uk.MMT4D_TYPE_S16S16S32,
               uk.MMT4D_TYPE_S8S4S32, uk.MMT4D_TYPE_F16F16F16, uk.MMT4D_TYPE_BF16BF16BF16]


def test_mmt4d_random_sweep(gpu, oracle):
    """Inputs are small integers (exact in every type), so any summation order
    must give the oracle's bits; tile shapes include ones no MFMA kernel takes."""
    lib, torch = gpu
    rng = np.random.default_rng(2026)
    kernels = set()
    for ci in range(180):
        tf = MMT4D_TYPES[ci % len(MMT4D_TYPES)]
        lb = uk.MMT4D_TYPE_BITS[tf][0]
        rbits = uk.MMT4D_TYPE_BITS[tf][1]
        M0, N0 = int(rng.choice([1, 2, 4, 8, 16, 24, 32, 64])), int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        K0 = int(rng.choice([1, 2, 4, 8, 16, 32]))
        if rbits == 4:
            K0 = max(2, K0)
        if tf == uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32:
            K0 = max(16, K0)
        M, N, K = int(rng.integers(0, 12)), int(rng.integers(0, 12)), int(rng.integers(0, 40))
        extra = uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS if rng.integers(0, 2) and lb == 16 else 0
        acc = uk.MMT4D_ACCUMULATE if rng.integers(0, 2) else 0
        slack = int(rng.choice([0, 16]))
        c = T.Mmt4dCase(tf | extra | acc, M, N, K, M0, N0, K0, K * M0 * K0 + slack,
                        K * N0 * K0 + slack, N * M0 * N0 + slack, slack, 0, slack)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want), (ci, c, lib.last_kernel_name())
        kernels.add(lib.last_kernel_name())
    assert "mmt4d_generic" in kernels and any(k.startswith("mmt4d_mfma") for k in kernels), kernels


def test_mmt4d_random_sweep_larger_shapes_and_forced_variants(gpu, oracle):
    """Tile counts large enough for the 128x128 / 256x256 workgroup shapes
    (several workgroups, ragged against them), a random forced variant per
    case, MFMA-served tile shapes only (incl. heights that do not divide the
    workgroup tile), K with and without a remainder against the pipeline step."""
    lib, torch = gpu
    rng = np.random.default_rng(2027)
    types = [uk.MMT4D_TYPE_S8S8S32, uk.MMT4D_TYPE_F16F16F32, uk.MMT4D_TYPE_BF16BF16F32,
             uk.MMT4D_TYPE_F32F32F32, uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32]
    done = 0
    for ci in range(300):
        tf = types[ci % len(types)]
        eb = uk.MMT4D_TYPE_BITS[tf][0] // 8
        M0, N0 = int(rng.choice([4, 8, 12, 16, 24, 32, 48, 64])), int(rng.choice([4, 8, 16, 20, 32, 64]))
        K0 = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        if not lib.mmt4d_info(M0, N0, K0, tf):
            continue
        M, N = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        K = int(rng.integers(1, max(2, 600 // (K0 * eb))))
        acc = uk.MMT4D_ACCUMULATE if rng.integers(0, 2) else 0
        c = T.Mmt4dCase(tf | acc, M, N, K, M0, N0, K0, K * M0 * K0 + 16, K * N0 * K0,
                        N * M0 * N0 + 16, 16, 0, 0)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        variant = int(rng.integers(0, 9))
        lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (ci, c, variant, lib.last_kernel_name())
        assert lib.last_kernel_name().startswith("mmt4d_mfma"), (ci, c, lib.last_kernel_name())
        done += 1
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    assert done >= 90, done


def test_mmt4d_random_sweep_lds_direct_pipeline(gpu, oracle):
    """The LDS-direct ping-pong pipeline (forced shapes 16 to 20): tile rows of
    2 to 64 bytes, random tiles incl. heights that straddle the 16-row MFMA
    blocks, tile counts ragged against the workgroup blocks, K with and
    without a remainder against the 64- or 256-byte step, loose strides, ACCUMULATE."""
    lib, torch = gpu
    rng = np.random.default_rng(2031)
    types = [uk.MMT4D_TYPE_S8S8S32, uk.MMT4D_TYPE_F16F16F32, uk.MMT4D_TYPE_BF16BF16F32,
             uk.MMT4D_TYPE_F32F32F32, uk.MMT4D_TYPE_F16F16F16 | uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS,
             uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32]
    names = set()
    done = 0
    for ci in range(210):
        tf = types[ci % len(types)]
        eb = uk.MMT4D_TYPE_BITS[tf & 0xFF][0] // 8
        M0, N0 = int(rng.choice([4, 8, 12, 16, 24, 32, 48, 64])), int(rng.choice([4, 8, 16, 20, 32, 64]))
        K0 = int(rng.choice([2, 4, 8, 16, 32, 64])) // eb
        if K0 < 1 or not lib.mmt4d_info(M0, N0, K0, tf):
            continue
        M, N = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        K = int(rng.integers(1, max(2, 1200 // (K0 * eb))))
        acc = uk.MMT4D_ACCUMULATE if rng.integers(0, 2) else 0
        c = T.Mmt4dCase(tf | acc, M, N, K, M0, N0, K0, K * M0 * K0 + 16, K * N0 * K0,
                        N * M0 * N0 + 16, 16, 0, 0)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + 16 + (ci // len(types)) % 5)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (ci, c, lib.last_kernel_name())
        names.add(lib.last_kernel_name())
        done += 1
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    assert done >= 70, done
    assert {"mmt4d_mfma_256x256_lds_direct", "mmt4d_mfma_128x512_lds_direct",
            "mmt4d_mfma_128x128_lds_direct", "mmt4d_mfma_64x64_lds_direct",
            "mmt4d_mfma_256x128_lds_direct"} <= names, names


def test_mmt4d_random_sweep_thin_kernels(gpu, oracle):
    """The barrier-free kernels (M-thin, N-thin on the transposed problem, the
    64x64 K split, the 4-bit RHS): K in whole 64- or 128-byte steps, few rows
    or few columns or few blocks, random tiles incl. heights that straddle the
    16-row MFMA blocks, loose strides, ACCUMULATE, each forced shape."""
    lib, torch = gpu
    rng = np.random.default_rng(2029)
    types = [uk.MMT4D_TYPE_S8S8S32, uk.MMT4D_TYPE_F16F16F32, uk.MMT4D_TYPE_BF16BF16F32,
             uk.MMT4D_TYPE_F32F32F32, uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, uk.MMT4D_TYPE_S8S4S32,
             uk.MMT4D_TYPE_F16F16F16 | uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS]
    names = set()
    done = 0
    for ci in range(420):
        tf = types[ci % len(types)]
        s8s4 = (tf & 0xFF) == uk.MMT4D_TYPE_S8S4S32
        bits = uk.MMT4D_TYPE_BITS[tf & 0xFF][0]
        M0, N0 = int(rng.choice([1, 2, 5, 8, 12, 16, 24, 32, 64])), int(rng.choice([1, 4, 8, 16, 20, 32, 64]))
        K0 = int(rng.choice([16, 32, 64] if s8s4 else [1, 2, 4, 8, 16, 32, 64]))
        rb = K0 * bits // 8
        if rb < 8 or rb > 128 or (not s8s4 and not lib.mmt4d_info(M0, N0, K0, tf)):
            continue
        step = 128 if (tf & 0xFF) == uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32 else 64
        if rb > step:
            continue
        K = (step // rb) * int(rng.integers(1, 9))             # whole steps
        shape_kind = ci % 3
        if shape_kind == 0:      # few rows
            M, N = max(1, int(rng.integers(1, 70)) // M0), int(rng.integers(1, 30))
        elif shape_kind == 1:    # few columns
            M, N = int(rng.integers(1, 30)), max(1, int(rng.integers(1, 70)) // N0)
        else:                    # a few blocks each way
            M, N = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        acc = uk.MMT4D_ACCUMULATE if rng.integers(0, 2) else 0
        c = T.Mmt4dCase(tf | acc, M, N, K, M0, N0, K0, K * M0 * K0 + 32, K * N0 * K0 + 32,
                        N * M0 * N0 + 16, 32, 32, 16)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        variant = 0 if s8s4 else int(rng.choice([0, 4, 5, 6]))
        lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want), (ci, c, variant, lib.last_kernel_name())
        assert lib.last_kernel_name().startswith("mmt4d_mfma"), (ci, c, variant, lib.last_kernel_name())
        names.add(lib.last_kernel_name())
        done += 1
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    assert done >= 150, done
    for want_name in ("mmt4d_mfma_thin", "mmt4d_mfma_thin_transposed", "mmt4d_mfma_64x64_ksplit",
                      "mmt4d_mfma_thin_s8s4"):
        assert want_name in names, names


def test_pack_unpack_random_round_trips_multi_block(gpu):
    """Sizes of several blocks per dimension: pack must equal numpy's
    pad + reshape + transpose and unpack must invert it, for random tiles,
    transposes and ragged sizes."""
    lib, torch = gpu
    rng = np.random.default_rng(2028)
    for ci in range(40):
        dtype, tf = [(np.float32, uk.PACK_TYPE_F32F32), (np.int8, uk.PACK_TYPE_I8I8),
                     (np.float16, uk.PACK_TYPE_F16F16), (np.int32, uk.PACK_TYPE_I32I32)][ci % 4]
        t0, t1 = int(rng.choice([1, 4, 8, 16, 32])), int(rng.choice([1, 2, 8, 16, 32]))
        ti, to = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        shape = (int(rng.integers(1, 700)), int(rng.integers(1, 700)))
        x = rng.integers(-100, 100, shape).astype(dtype)
        pad_val = dtype(-3)
        pad_bits = int(np.array([pad_val]).view({1: np.uint8, 2: np.uint16, 4: np.uint32}[x.itemsize])[0])
        want4 = T.numpy_pack(x, t0, t1, ti, to, pad_val)
        o0, o1, o2, o3 = want4.shape
        d_x = torch.from_numpy(x).cuda()
        d_p = torch.zeros(want4.size * x.itemsize, dtype=torch.uint8, device="cuda")
        flags = tf | (0x100 if ti else 0) | (0x200 if to else 0)
        lib.pack(d_x.data_ptr(), 0, shape[1], 1, d_p.data_ptr(), 0, o1 * o2 * o3, o2 * o3, shape[0],
                 shape[1], o0, o1, o2, o3, pad_bits, flags)
        got4 = d_p.cpu().numpy().view(dtype).reshape(want4.shape)
        assert np.array_equal(got4, want4), (ci, shape, t0, t1, ti, to, lib.last_kernel_name())
        if tf == uk.PACK_TYPE_I8I8:
            continue  # unpack has no 1-byte type
        d_y = torch.full((x.size * x.itemsize,), 0x5A, dtype=torch.uint8, device="cuda")
        lib.unpack(d_p.data_ptr(), 0, o1 * o2 * o3, o2 * o3, d_y.data_ptr(), 0, shape[1], 1, o0, o1,
                   o2, o3, shape[0], shape[1], flags)
        back = d_y.cpu().numpy().view(dtype).reshape(shape)
        assert np.array_equal(back, x), (ci, shape, t0, t1, ti, to, lib.last_kernel_name())


def test_mmt4d_random_sweep_narrow_row_kernels(gpu, oracle):
    """The narrow-row kernels (tile rows of 2 or 4 bytes, N0 = 16: the RHS is
    read straight into registers with its rows permuted across accumulator
    blocks, the LHS loader waves take the steps in turns): random tile heights,
    tile counts ragged against every workgroup shape, K with and without a
    remainder against the 64-byte step, ACCUMULATE, loose strides, in every
    shape the kernel is built in (12 .. 15) and as the library chooses (0)."""
    lib, torch = gpu
    rng = np.random.default_rng(4242)
    tiles = [(uk.MMT4D_TYPE_S8S8S32, 2), (uk.MMT4D_TYPE_S8S8S32, 4), (uk.MMT4D_TYPE_F16F16F32, 1),
             (uk.MMT4D_TYPE_F16F16F32, 2), (uk.MMT4D_TYPE_BF16BF16F32, 2), (uk.MMT4D_TYPE_BF16BF16F32, 1),
             (uk.MMT4D_TYPE_F32F32F32, 1)]
    served = set()
    for ci in range(196):
        tf, K0 = tiles[ci % len(tiles)]
        rb = K0 * uk.MMT4D_TYPE_BITS[tf][0] // 8
        M0 = int(rng.choice([8, 16, 24, 32, 64]))
        M, N = int(rng.integers(1, 48)), int(rng.integers(1, 48))
        K = int(rng.integers(1, 900 // rb))
        if ci % 5 == 0:
            K = (K // (64 // rb) + 1) * (64 // rb)          # whole steps only
        acc = uk.MMT4D_ACCUMULATE if rng.integers(0, 2) else 0
        slack = 16 * int(rng.integers(0, 2))
        c = T.Mmt4dCase(tf | acc, M, N, K, M0, 16, K0, K * M0 * K0 + slack, K * 16 * K0 + slack,
                        N * M0 * 16 + slack, slack, 0, slack)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        variant = int(rng.choice([0, 12, 13, 14, 15]))
        lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert np.array_equal(got, want), (ci, c, variant, lib.last_kernel_name())
        served.add(lib.last_kernel_name())
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    for shape in ("256x256", "128x512", "128x128", "64x64"):
        assert f"mmt4d_mfma_{shape}_narrow" in served, served
