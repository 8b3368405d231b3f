"""GPU parity of iree_uk_pack / iree_uk_unpack against the CPU oracle, through
the C-ABI. Bit-exact over the whole destination buffer (stride gaps must stay
untouched)."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

MODES = [uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_GENERIC]


@pytest.fixture(autouse=True)
def _reset_modes(lib):
    yield
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_pointer_mode(uk.POINTER_MODE_AUTO)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("n", range(len(G.PACK_TILES)))
def test_pack_reference_test_grid(gpu, oracle, n, mode):
    """tools/pack_test.c's grid: degenerate and small outer shapes x both
    transposes x padding variants, random strides/offsets/padding value."""
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    tf, t0, t1 = G.PACK_TILES[n]
    for ci, c in enumerate(T.pack_cases(tf, t0, t1, seed=11000 + n)):
        rng = np.random.default_rng(ci)
        inp, out0 = T.make_pack_buffers(c, rng)
        want = out0.copy()
        G.run_pack_case(oracle, c, inp, want)
        got = T.gpu_pack(lib, torch, c, inp, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("n", range(len(G.UNPACK_TILES)))
def test_unpack_reference_test_grid(gpu, oracle, n, mode):
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    tf, t0, t1 = G.UNPACK_TILES[n]
    for ci, c in enumerate(T.unpack_cases(tf, t0, t1, seed=12000 + n)):
        rng = np.random.default_rng(ci)
        inp, out0 = T.make_unpack_buffers(c, rng)
        want = out0.copy()
        G.run_unpack_case(oracle, c, inp, want)
        got = T.gpu_unpack(lib, torch, c, inp, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())


# Shapes large enough to span several workgroup blocks of the tiled kernels,
# with ragged edges, all-padding tiles, loose strides and shifted bases.
TILED_SHAPES = [
    # (type, tile0, tile1, in0, in1)
    (uk.PACK_TYPE_F16F16, 16, 16, 300, 270),
    (uk.PACK_TYPE_F16F16, 16, 16, 256, 256),
    (uk.PACK_TYPE_I8I8, 16, 32, 130, 515),
    (uk.PACK_TYPE_I8I8, 32, 8, 16, 1024),
    (uk.PACK_TYPE_I8I8, 16, 2, 200, 301),
    (uk.PACK_TYPE_I8I8, 16, 8, 257, 259),
    (uk.PACK_TYPE_F32F32, 16, 1, 259, 263),
    (uk.PACK_TYPE_F32F32, 16, 16, 100, 333),
    (uk.PACK_TYPE_I32I32, 8, 4, 77, 130),
    (uk.PACK_TYPE_BF16BF16, 16, 2, 130, 258),
    (uk.PACK_TYPE_F16F16, 1, 16, 37, 400),
    (uk.PACK_TYPE_F32F32, 3, 5, 200, 200),
    (uk.PACK_TYPE_F16F16, 6, 7, 200, 200),
]


def _tiled_pack_cases():
    g = T.Lcg(77)
    for (tf, t0, t1, in0, in1) in TILED_SHAPES:
        for ti in (0, 1):
            for to in (0, 1):
                for variant in range(3):
                    a0, a1 = (t1, t0) if ti else (t0, t1)  # extent along matrix dims
                    o0 = -(-in0 // a0) + (1 if variant == 2 else 0)
                    o1 = -(-in1 // a1) + (2 if variant == 2 else 0)
                    flags = tf | (0x100 if ti else 0) | (0x200 if to else 0)
                    os0, os1 = (o1, o0) if to else (o0, o1)
                    loose = (0, 4, 1)[variant]
                    yield T.PackCase(flags, in0, in1, os0, os1, t0, t1,
                                     in1 + (0, 8, 3)[variant], 1,
                                     os1 * t0 * t1 + loose,
                                     (0, 16, 5)[variant], (0, 32, 3)[variant], g.u64())


@pytest.mark.parametrize("mode", MODES)
def test_pack_block_spanning_shapes(gpu, oracle, mode):
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    tiled = 0
    for ci, c in enumerate(_tiled_pack_cases()):
        rng = np.random.default_rng(500 + ci)
        inp, out0 = T.make_pack_buffers(c, rng)
        want = out0.copy()
        G.run_pack_case(oracle, c, inp, want)
        got = T.gpu_pack(lib, torch, c, inp, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        tiled += lib.last_kernel_name() in ("pack_tiled", "pack_stream", "pack_direct", "pack_transposing")
    if mode == uk.KERNEL_MODE_AUTO:
        assert tiled >= 60, tiled  # the LDS-staged kernel is the one under test
    else:
        assert tiled == 0


@pytest.mark.parametrize("mode", MODES)
def test_unpack_block_spanning_shapes(gpu, oracle, mode):
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    tiled = 0
    for ci, pc in enumerate(_tiled_pack_cases()):
        if pc.elem_bytes == 1:
            continue  # unpack has no 1-byte type (exported_bits.h:76)
        c = T.UnpackCase(pc.flags, pc.out_size0, pc.out_size1, pc.out_size2,
                         pc.out_size3, pc.in_size0, pc.in_size1, pc.out_stride0,
                         pc.in_stride0, 1, pc.out_offset, pc.in_offset)
        rng = np.random.default_rng(900 + ci)
        inp, out0 = T.make_unpack_buffers(c, rng)
        want = out0.copy()
        G.run_unpack_case(oracle, c, inp, want)
        got = T.gpu_unpack(lib, torch, c, inp, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        tiled += lib.last_kernel_name() in ("unpack_tiled", "unpack_stream")
    if mode == uk.KERNEL_MODE_AUTO:
        assert tiled >= 40, tiled


@pytest.mark.parametrize("tf,t0,t1", [
    (uk.PACK_TYPE_I8I8, 16, 16), (uk.PACK_TYPE_I8I8, 16, 32), (uk.PACK_TYPE_I8I8, 32, 64),
    (uk.PACK_TYPE_I8I8, 1, 128), (uk.PACK_TYPE_F16F16, 16, 16), (uk.PACK_TYPE_BF16BF16, 24, 8),
    (uk.PACK_TYPE_F32F32, 8, 4), (uk.PACK_TYPE_I32I32, 5, 16)])
def test_pack_direct_kernel_exact_untransposed_tilings(gpu, oracle, tf, t0, t1):
    """Untransposed packs of a matrix that the tiles cover exactly, tile rows of
    whole 16-byte pieces, 16-byte aligned rows: the register-to-register kernel
    (no LDS staging) serves them up to a few tens of megabytes. Whole output
    buffers against the oracle, loose pitches and offsets included, and the
    LDS-staged kernels on the same call give the same bytes."""
    lib, torch = gpu
    es = uk.PACK_TYPE_BYTES[tf]
    align = 16 // es
    for ci, (o0, o1) in enumerate(((1, 1), (3, 5), (17, 9), (40, 33), (2, 130))):
        in0, in1 = o0 * t0, o1 * t1
        c = T.PackCase(tf, in0, in1, o0, o1, t0, t1, in1 + (ci % 3) * align, 1,
                       o1 * t0 * t1 + (ci % 2) * align, (ci % 2) * align, (ci % 3) * align, 0x1234)
        rng = np.random.default_rng(7000 + ci)
        inp, out0 = T.make_pack_buffers(c, rng)
        want = out0.copy()
        G.run_pack_case(oracle, c, inp, want)
        lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        got = T.gpu_pack(lib, torch, c, inp, out0)
        assert lib.last_kernel_name() == "pack_direct", (c.label(), lib.last_kernel_name())
        assert np.array_equal(got, want), c.label()
        lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + 1)   # keeps pack on the LDS-staged kernels
        try:
            staged = T.gpu_pack(lib, torch, c, inp, out0)
            assert lib.last_kernel_name() in ("pack_stream", "pack_tiled"), lib.last_kernel_name()
        finally:
            lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        assert np.array_equal(staged, want), c.label()


# (type, stored tile shape out_size2 x out_size3, TRANSPOSE_INNER): element-wise
# transpositions, and untransposed tiles whose rows are one, two or four bytes
# (the reference's 16x2 s8 tile,
# arch/x86_64/mmt4d_x86_64_tiles.inl).
TRANSPOSING_TILES = [
    (uk.PACK_TYPE_F16F16, 16, 16, True), (uk.PACK_TYPE_BF16BF16, 16, 8, True), (uk.PACK_TYPE_F16F16, 16, 4, True),
    (uk.PACK_TYPE_F16F16, 64, 32, True), (uk.PACK_TYPE_F16F16, 1, 16, True), (uk.PACK_TYPE_BF16BF16, 128, 16, True),
    (uk.PACK_TYPE_I8I8, 16, 8, True), (uk.PACK_TYPE_I8I8, 16, 16, True), (uk.PACK_TYPE_I8I8, 16, 32, True),
    (uk.PACK_TYPE_I8I8, 8, 32, True), (uk.PACK_TYPE_I8I8, 256, 8, True), (uk.PACK_TYPE_I8I8, 2, 16, True),
    (uk.PACK_TYPE_I8I8, 16, 2, False), (uk.PACK_TYPE_I8I8, 8, 2, False), (uk.PACK_TYPE_I8I8, 32, 2, False),
    (uk.PACK_TYPE_I8I8, 16, 1, False), (uk.PACK_TYPE_I8I8, 8, 1, False),
    (uk.PACK_TYPE_F16F16, 16, 1, False), (uk.PACK_TYPE_BF16BF16, 4, 1, False),
    # transposed tiles less than eight bytes tall (K0 = 2 and 4 from a row-major [K][N] operand)
    (uk.PACK_TYPE_I8I8, 16, 2, True), (uk.PACK_TYPE_I8I8, 16, 4, True), (uk.PACK_TYPE_BF16BF16, 16, 2, True),
    (uk.PACK_TYPE_I8I8, 8, 2, True), (uk.PACK_TYPE_F16F16, 8, 2, True), (uk.PACK_TYPE_I8I8, 4, 4, True),
    (uk.PACK_TYPE_I8I8, 256, 2, True),
    # four-byte elements: f32 / s32 tiles one element wide, 16-bit pairs and s8 quadruples as tile rows
    # (the reference's 16x16x1 f32 and 16x16x2 bf16 tiles on x86, 8x8x4 s8 on arm64), and f32 transposed
    (uk.PACK_TYPE_F32F32, 16, 1, False), (uk.PACK_TYPE_I32I32, 8, 1, False), (uk.PACK_TYPE_F32F32, 4, 1, False),
    (uk.PACK_TYPE_F32F32, 32, 1, False), (uk.PACK_TYPE_BF16BF16, 16, 2, False), (uk.PACK_TYPE_F16F16, 8, 2, False),
    (uk.PACK_TYPE_I8I8, 16, 4, False), (uk.PACK_TYPE_I8I8, 8, 4, False),
    (uk.PACK_TYPE_F32F32, 16, 4, True), (uk.PACK_TYPE_F32F32, 8, 8, True), (uk.PACK_TYPE_I32I32, 64, 16, True), (uk.PACK_TYPE_F16F16, 8, 32, True),
]


def _transposing_cases(tf, s2, s3, ti):
    """Matrix shapes around the kernel's 32-row x 512-byte blocks: one block and
    less, several with ragged edges in both directions, tile grids larger than
    the matrix (tiles of nothing but padding), both outer orders, loose pitches
    and offsets that keep the alignment the kernel asks for (4 bytes on the
    matrix side, 16 on the tiled side)."""
    es = uk.PACK_TYPE_BYTES[tf]
    a0, a1 = (s3, s2) if ti else (s2, s3)    # tile extent along matrix rows / columns
    g = T.Lcg(1234 + s2 * 7 + s3)
    even = 1 if ti else s3                   # (whole tile rows)
    for (in0, in1, extra) in ((5, 6, 0), (32, 512 // es, 0), (67, 2 * (512 // es) + 10, 0), (200, 130, 1),
                              (129, 700, 0), (3 * 32, 3 * (512 // es), 2)):
        in1 = -(-in1 // even) * even
        for to in (0, 1):
            for variant in range(2):
                o0 = -(-in0 // a0) + extra
                o1 = -(-in1 // a1) + (extra + 1) // 2
                os0, os1 = (o1, o0) if to else (o0, o1)
                flags = tf | (0x100 if ti else 0) | (0x200 if to else 0)
                unit = 16 // es
                yield T.PackCase(flags, in0, in1, os0, os1, s2, s3,
                                 -(-in1 // 4) * 4 + (0, 4 * 3)[variant], 1,
                                 os1 * s2 * s3 + (0, unit * 3)[variant],
                                 (0, 4 * 5)[variant], (0, unit * 2)[variant], g.u64())


@pytest.mark.parametrize("tile", TRANSPOSING_TILES, ids=lambda t: f"type{t[0]}_{t[1]}x{t[2]}_{'ti' if t[3] else 'rows'}")
def test_pack_transposing_kernel(gpu, oracle, tile):
    """The kernel built on the LDS transposing reads: whole output buffers
    against the oracle, and the LDS-staged kernels on the same calls."""
    lib, torch = gpu
    tf, s2, s3, ti = tile
    for ci, c in enumerate(_transposing_cases(tf, s2, s3, ti)):
        rng = np.random.default_rng(8000 + ci)
        inp, out0 = T.make_pack_buffers(c, rng)
        want = out0.copy()
        G.run_pack_case(oracle, c, inp, want)
        lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        got = T.gpu_pack(lib, torch, c, inp, out0)
        assert lib.last_kernel_name() == "pack_transposing", (c.label(), lib.last_kernel_name())
        assert np.array_equal(got, want), c.label()
        lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + 1)   # keeps pack on the LDS-staged kernels
        try:
            staged = T.gpu_pack(lib, torch, c, inp, out0)
            assert lib.last_kernel_name() in ("pack_stream", "pack_tiled"), lib.last_kernel_name()
        finally:
            lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        assert np.array_equal(staged, want), c.label()


def test_pack_transposing_kernel_declines_what_it_does_not_serve(gpu, oracle):
    """Rows that are only 2-byte aligned, tile extents that are not powers of
    two, an odd number of columns under two-byte tile rows, four-byte elements
    in tiles less than 16 bytes tall: other kernels, same bytes."""
    lib, torch = gpu
    cases = [T.PackCase(uk.PACK_TYPE_F16F16 | 0x100, 70, 131, 5, 9, 16, 16, 131, 1, 9 * 256, 0, 0, 7),
             T.PackCase(uk.PACK_TYPE_I8I8 | 0x100, 70, 130, 6, 6, 24, 12, 132, 1, 6 * 288, 0, 0, 7),
             T.PackCase(uk.PACK_TYPE_I8I8, 70, 131, 5, 66, 16, 2, 132, 1, 66 * 32, 0, 0, 7),
             T.PackCase(uk.PACK_TYPE_F32F32 | 0x100, 70, 130, 35, 9, 16, 2, 132, 1, 9 * 32, 0, 0, 7),
             T.PackCase(uk.PACK_TYPE_F32F32, 70, 130, 35, 130, 2, 1, 132, 1, 130 * 2, 0, 0, 7)]
    for ci, c in enumerate(cases):
        inp, out0 = T.make_pack_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_pack_case(oracle, c, inp, want)
        got = T.gpu_pack(lib, torch, c, inp, out0)
        assert lib.last_kernel_name() != "pack_transposing", c.label()
        assert np.array_equal(got, want), c.label()


SINGLE_LINE_TILES = [
    (uk.PACK_TYPE_F32F32, 16, 1), (uk.PACK_TYPE_F32F32, 1, 16), (uk.PACK_TYPE_I32I32, 8, 1),
    (uk.PACK_TYPE_F16F16, 1, 16), (uk.PACK_TYPE_BF16BF16, 16, 1), (uk.PACK_TYPE_I8I8, 1, 16),
    (uk.PACK_TYPE_I8I8, 16, 1), (uk.PACK_TYPE_F32F32, 1, 1), (uk.PACK_TYPE_F32F32, 1, 7),
]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("tile", SINGLE_LINE_TILES, ids=lambda t: f"type{t[0]}_{t[1]}x{t[2]}")
def test_single_row_and_single_column_tiles_under_transpose_inner(gpu, oracle, tile, mode):
    """A tile that is one row or one column holds the same bytes with and without
    TRANSPOSE_INNER, and the library takes it as the untransposed tile of the
    swapped shape (the reference's f32 16x16x1 right-hand side packed from
    [K][N], arch/x86_64/mmt4d_x86_64_tiles.inl). Pack and unpack, both outer
    orders, ragged edges, loose pitches: whole buffers against the oracle."""
    lib, torch = gpu
    lib.set_kernel_mode(mode)
    tf, s2, s3 = tile
    es = uk.PACK_TYPE_BYTES[tf]
    a0, a1 = s3, s2                       # TRANSPOSE_INNER: extents along matrix rows / columns
    g = T.Lcg(77 + 3 * s2 + s3)
    ci = 0
    for (in0, in1) in ((1, 1), (33, 70), (130, 257), (64, 512)):
        for to in (0, 1):
            for variant in range(2):
                o0, o1 = -(-in0 // a0) + variant, -(-in1 // a1)
                os0, os1 = (o1, o0) if to else (o0, o1)
                flags = tf | 0x100 | (0x200 if to else 0)
                c = T.PackCase(flags, in0, in1, os0, os1, s2, s3, in1 + (0, 5)[variant], 1,
                               os1 * s2 * s3 + (0, 3)[variant], (0, 2)[variant], (0, 9)[variant], g.u64())
                inp, out0 = T.make_pack_buffers(c, np.random.default_rng(4100 + ci))
                want = out0.copy()
                G.run_pack_case(oracle, c, inp, want)
                got = T.gpu_pack(lib, torch, c, inp, out0)
                assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
                if es > 1:                # unpack has no 1-byte type (exported_bits.h:76)
                    u = T.UnpackCase(flags, os0, os1, s2, s3, in0, in1, c.out_stride0, c.in_stride0, 1,
                                     c.out_offset, c.in_offset)
                    uin, uout0 = T.make_unpack_buffers(u, np.random.default_rng(4200 + ci))
                    uwant = uout0.copy()
                    G.run_unpack_case(oracle, u, uin, uwant)
                    ugot = T.gpu_unpack(lib, torch, u, uin, uout0)
                    assert np.array_equal(ugot, uwant), (u.label(), lib.last_kernel_name())
                ci += 1


def test_pack_unpack_round_trip_and_numpy_identity(gpu):
    """Size-independent properties at a size the oracle would be slow on:
    pack == pad+reshape+transpose, unpack(pack(x)) == x."""
    lib, torch = gpu
    rng = np.random.default_rng(1)
    for (dtype, tf, t0, t1, ti, to, shape) in (
            (np.float32, uk.PACK_TYPE_F32F32, 16, 1, False, True, (1537, 1030)),
            (np.float16, uk.PACK_TYPE_F16F16, 16, 16, False, False, (2047, 2049)),
            (np.int32, uk.PACK_TYPE_I32I32, 16, 16, True, True, (1000, 999)),
            # above 192 MB: the 64 KB-block kernels for large element-granular
            # transposes, with rows that are only 4-byte aligned and ragged edges
            (np.float32, uk.PACK_TYPE_F32F32, 16, 1, False, True, (7169, 7171)),
            # above 192 MB with whole tile rows as granules under TRANSPOSE_OUTER:
            # the 16 KB-block kernels with their non-temporal stores
            (np.float32, uk.PACK_TYPE_F32F32, 16, 16, False, True, (8192, 8192 - 16))):
        x = rng.integers(-30000, 30000, shape).astype(dtype)
        pad_val = dtype(-1)
        pad_bits = int(np.array([pad_val]).view({2: np.uint16, 4: np.uint32}[x.itemsize])[0])
        want4 = T.numpy_pack(x, t0, t1, ti, to, pad_val)
        o0, o1, o2, o3 = want4.shape
        d_x = torch.from_numpy(x).cuda()
        d_p = torch.zeros(want4.size * x.itemsize, dtype=torch.uint8, device="cuda")
        flags = tf | (0x100 if ti else 0) | (0x200 if to else 0)
        lib.pack(d_x.data_ptr(), 0, shape[1], 1, d_p.data_ptr(), 0, o1 * o2 * o3,
                 o2 * o3, shape[0], shape[1], o0, o1, o2, o3, pad_bits, flags)
        assert lib.last_kernel_name() in ("pack_stream", "pack_tiled", "pack_direct", "pack_transposing")
        got4 = d_p.cpu().numpy().view(dtype).reshape(want4.shape)
        assert np.array_equal(got4, want4)
        d_y = torch.full((x.size * x.itemsize,), 0x5A, dtype=torch.uint8, device="cuda")
        lib.unpack(d_p.data_ptr(), 0, o1 * o2 * o3, o2 * o3, d_y.data_ptr(), 0,
                   shape[1], 1, o0, o1, o2, o3, shape[0], shape[1], flags)
        assert lib.last_kernel_name() in ("unpack_stream", "unpack_tiled")
        assert np.array_equal(d_y.cpu().numpy().view(dtype).reshape(shape), x)


def test_host_pointers_are_staged(gpu, oracle):
    """Ordinary host memory works through the same entry points (staged through
    the GPU) and leaves stride gaps of the destination untouched."""
    lib, torch = gpu
    for ci, c in enumerate(T.pack_cases(uk.PACK_TYPE_F16F16, 6, 7, seed=31,
                                        outer_shapes=((3, 2), (9, 33)), max_offset=64)):
        rng = np.random.default_rng(ci)
        inp, out0 = T.make_pack_buffers(c, rng)
        want = out0.copy()
        G.run_pack_case(oracle, c, inp, want)
        got = out0.copy()
        es = c.elem_bytes
        lib.pack(inp.ctypes.data - c.in_offset * es, c.in_offset, c.in_stride0,
                 c.in_stride1, got.ctypes.data - c.out_offset * es, c.out_offset,
                 c.out_stride0, c.out_stride1, c.in_size0, c.in_size1, c.out_size0,
                 c.out_size1, c.out_size2, c.out_size3, c.padding_value, c.flags)
        assert np.array_equal(got, want), c.label()
    for ci, c in enumerate(T.unpack_cases(uk.UNPACK_TYPE_I32I32, 3, 4, seed=32,
                                          outer_shapes=((3, 2), (9, 33)), max_offset=64)):
        rng = np.random.default_rng(ci)
        inp, out0 = T.make_unpack_buffers(c, rng)
        want = out0.copy()
        G.run_unpack_case(oracle, c, inp, want)
        got = out0.copy()
        es = c.elem_bytes
        lib.unpack(inp.ctypes.data - c.in_offset * es, c.in_offset, c.in_stride0,
                   c.in_stride1, got.ctypes.data - c.out_offset * es, c.out_offset,
                   c.out_stride0, c.out_stride1, c.in_size0, c.in_size1, c.in_size2,
                   c.in_size3, c.out_size0, c.out_size1, c.flags)
        assert np.array_equal(got, want), c.label()
