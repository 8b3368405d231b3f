"""K split over workgroups in the M-thin / N-thin mmt4d kernels (decode-shaped
problems with too few output blocks to occupy the chip): every slice count
against the CPU oracle, through the C-ABI. Integer types bit-exact; float types
bit-exact too, on the small-integer inputs of the reference's own tests
(tools/util.c:131-165: every partial sum is exact, so neither the split nor the
order in which the slices are added can show)."""
import numpy as np
import pytest

import uk_testing as T
from golden import make_golden as G
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

TILES = [(uk.MMT4D_TYPE_S8S8S32, 32, 16, 8), (uk.MMT4D_TYPE_S8S8S32, 16, 16, 16),
         (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16), (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 8),
         (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, 16, 16, 32), (uk.MMT4D_TYPE_F32F32F32, 16, 16, 4),
         (uk.MMT4D_TYPE_S8S4S32, 16, 16, 32)]


@pytest.fixture(autouse=True)
def _reset(lib):
    yield
    lib.set_k_slices(0)
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)


# (tile, N-thin?): the 4-bit RHS kernel serves M-thin problems only.
CASES = [(t, n_thin) for t in TILES for n_thin in (False, True)
         if not (n_thin and t[0] == uk.MMT4D_TYPE_S8S4S32)]


@pytest.mark.parametrize("slices", [2, 3, 5])
@pytest.mark.parametrize("tile,n_thin", CASES)
def test_thin_kernels_with_k_slices(gpu, oracle, tile, n_thin, slices):
    lib, torch = gpu
    tf, M0, N0, K0 = tile
    lb = uk.MMT4D_TYPE_BITS[tf][0]
    step_elems = (128 if tf == uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32 else 64) * 8 // lb
    # Each wave keeps at least four steps: 16 steps per slice, plus a few so
    # that the slices are not all the same length.
    k_tiles = (16 * slices + 3) * step_elems // K0
    thin, wide = (1, 7)
    shape = (wide, thin, k_tiles) if n_thin else (thin, wide, k_tiles)
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_k_slices(slices)
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=4300 + slices, slack=16, shapes=(shape,))):
        rng = np.random.default_rng(900 + ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        assert lib.last_kernel_name().startswith("mmt4d_mfma_thin"), lib.last_kernel_name()
        assert lib.last_k_slices() == slices


def test_k_slices_are_chosen_for_a_decode_step_with_few_columns(gpu):
    """A decode step against a weight matrix of few rows and a long K (16 rows,
    K = 14336, N = 1024, tiles 32x16x8, ACCUMULATE): 64 output blocks of 16
    columns for 256 compute units. The library splits K on its own, and the
    result is the exact integer product plus the initial accumulators."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_k_slices(0)
    Mlog, K, N, M0, N0, K0 = 16, 14336, 1024, 32, 16, 8
    N1, K1 = N // N0, K // K0
    g = torch.Generator(device="cuda"); g.manual_seed(41)
    act = torch.randint(-128, 128, (Mlog, K), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (N, K), generator=g, device="cuda", dtype=torch.int8)
    lhs4 = torch.zeros(K1 * M0 * K0, device="cuda", dtype=torch.int8)
    rhs4 = torch.zeros(N1 * K1 * N0 * K0, device="cuda", dtype=torch.int8)
    lib.pack(act.data_ptr(), 0, K, 1, lhs4.data_ptr(), 0, K1 * M0 * K0, M0 * K0, Mlog, K, 1, K1, M0, K0, 0,
             uk.PACK_TYPE_I8I8)
    lib.pack(w.data_ptr(), 0, K, 1, rhs4.data_ptr(), 0, K1 * N0 * K0, N0 * K0, N, K, N1, K1, N0, K0, 0,
             uk.PACK_TYPE_I8I8)
    acc0 = torch.randint(-2 ** 15, 2 ** 15, (N1, M0, N0), generator=g, device="cuda", dtype=torch.int32)
    out4 = acc0.clone()
    lib.mmt4d(lhs4.data_ptr(), 0, K1 * M0 * K0, rhs4.data_ptr(), 0, K1 * N0 * K0, out4.data_ptr(), 0,
              N1 * M0 * N0, 1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_mfma_thin"
    assert lib.last_k_slices() > 1
    prod = act.cpu().to(torch.int64) @ w.cpu().to(torch.int64).T                       # [16][N]
    want = acc0.cpu().to(torch.int64)
    want[:, :Mlog, :] += prod.view(Mlog, N1, N0).permute(1, 0, 2)
    assert torch.equal(out4.cpu().to(torch.int64), want)


def test_k_slices_with_the_dequantizing_store(gpu):
    """The fused dequantizing call under a forced split equals the unsplit one
    bit for bit (integer accumulators: the split cannot show)."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    rows, K, N, M0, N0, K0 = 16, 4096, 512, 16, 16, 16
    N1, K1 = N // N0, K // K0
    g = torch.Generator(device="cuda"); g.manual_seed(43)
    lhs = torch.randint(-128, 128, (K1 * M0 * K0,), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1 * K1 * N0 * K0,), generator=g, device="cuda", dtype=torch.int8)
    acc = torch.randint(-1000, 1000, (N1 * M0 * N0,), generator=g, device="cuda", dtype=torch.int32)
    rs = torch.rand(rows, generator=g, device="cuda") * 0.02 + 0.001
    cs = torch.rand(N, generator=g, device="cuda") * 0.02 + 0.001
    results = []
    for slices in (1, 4):
        lib.set_k_slices(slices)
        y = torch.full((rows, N), -1.0, device="cuda")
        lib.mmt4d_dequant_unpack(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0,
                                 acc.data_ptr(), 0, N1 * M0 * N0, y.data_ptr(), 0, N, rows, N,
                                 rs.data_ptr(), cs.data_ptr(), 1, N1, K1, M0, N0, K0,
                                 uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE)
        lib.synchronize()
        assert lib.last_k_slices() == slices
        results.append(y)
    assert torch.equal(results[0], results[1])


def test_k_slices_on_the_32_column_blocks(gpu, oracle):
    """Enough columns for a 32-column block per compute unit (so the narrow
    16-column blocks are not chosen) and a forced split."""
    lib, torch = gpu
    tf, M0, N0, K0 = uk.MMT4D_TYPE_S8S8S32, 16, 16, 16
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_k_slices(2)
    for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=4400, slack=16, shapes=((1, 640, 35 * 4),))):
        rng = np.random.default_rng(950 + ci)
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, rng)
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0)
        assert np.array_equal(got, want), (c.label(), lib.last_kernel_name())
        assert lib.last_kernel_name() == "mmt4d_mfma_thin" and lib.last_k_slices() == 2


@pytest.mark.parametrize("n_thin", [False, True])
@pytest.mark.parametrize("tf,M0,N0,K0", [(uk.MMT4D_TYPE_S8S8S32, 32, 16, 8), (uk.MMT4D_TYPE_S8S8S32, 16, 16, 16),
                                         (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16), (uk.MMT4D_TYPE_S8S4S32, 16, 16, 32)])
def test_streamed_weights_hint_changes_no_result(gpu, tf, M0, N0, K0, n_thin):
    """iree_uk_amd_set_streamed_weights: the decode-shaped kernels then load
    weights of 16 MB and more non-temporally. Same bytes out as without the
    hint, thin in M and thin in N (the transposed problem), with and without a
    K split; and the hint is the calling thread's own, reset here."""
    lib, torch = gpu
    wide, K = 4608, 4096                      # 18.9 MB of 1-byte weights
    if tf == uk.MMT4D_TYPE_S8S4S32:
        wide *= 2                             # two elements per byte
    if n_thin and tf == uk.MMT4D_TYPE_S8S4S32:
        pytest.skip("the 4-bit operand is the right-hand side only")
    lhs_es = {uk.MMT4D_TYPE_F16F16F32: 2}.get(tf, 1)
    M1, N1 = (wide // M0, 1) if n_thin else (1, wide // N0)
    K1 = K // K0
    g = torch.Generator(device="cuda"); g.manual_seed(5)

    def operand(rows_tiles, X0, packed_nibbles=False):
        n = rows_tiles * K1 * X0 * K0
        if lhs_es == 2:
            return (torch.randint(-8, 8, (n,), generator=g, device="cuda", dtype=torch.int32)).to(torch.float16)
        if packed_nibbles:
            return torch.randint(-128, 128, (n // 2,), generator=g, device="cuda", dtype=torch.int8)
        return torch.randint(-128, 128, (n,), generator=g, device="cuda", dtype=torch.int8)

    lhs = operand(M1, M0)
    rhs = operand(N1, N0, packed_nibbles=tf == uk.MMT4D_TYPE_S8S4S32)
    out_dt = torch.float32 if lhs_es == 2 else torch.int32
    outs = []
    try:
        for hint, slices in ((False, 0), (True, 0), (True, 1)):
            lib.set_streamed_weights(hint)
            lib.set_k_slices(slices)
            out = torch.zeros(M1 * N1 * M0 * N0, device="cuda", dtype=out_dt)
            lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
                      N1 * M0 * N0, M1, N1, K1, M0, N0, K0, tf | 0x200)
            lib.synchronize()
            assert lib.last_kernel_name().startswith("mmt4d_mfma_thin"), lib.last_kernel_name()
            outs.append(out)
    finally:
        lib.set_streamed_weights(False)
        lib.set_k_slices(0)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert bool(outs[0].any())


@pytest.mark.gpu
@pytest.mark.parametrize("tf,K0", [(uk.MMT4D_TYPE_S8S8S32, 16), (uk.MMT4D_TYPE_F16F16F32, 8)])
def test_few_blocks_and_a_long_k_split_k_over_workgroups(gpu, oracle, tf, K0):
    """A small output against a long K (144 x 130 outputs, 32 KB of K per row):
    the 64x64 kernel, whose four waves already split K inside the workgroup,
    splits it over workgroups as well. Against the oracle on the reference
    tests' values (integers exact; float sums exact in any order), ACCUMULATE
    off and on, and more than one slice reported."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    bits = uk.MMT4D_TYPE_BITS[tf][0]
    K1 = 32768 * 8 // bits // K0
    for ci, c in enumerate(T.mmt4d_cases(tf, 16, 16, K0, seed=61, slack=16, shapes=((9, 9, K1),))):
        lhs, rhs, out0 = T.make_mmt4d_buffers(c, np.random.default_rng(ci))
        want = out0.copy()
        G.run_mmt4d_case(oracle, c, lhs, rhs, want)
        got = T.gpu_mmt4d(lib, torch, c, lhs, rhs, out0, allow_generic=False)
        assert lib.last_kernel_name() == "mmt4d_mfma_64x64_ksplit", lib.last_kernel_name()
        assert lib.last_k_slices() > 1
        assert np.array_equal(got, want), c.label()
