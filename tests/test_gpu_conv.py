"""conv_nchwc on the GPU against the oracle, through the C-ABI: the reference
test's case grid (tools/conv_nchwc_test.c:187-226; random loose strides and
offsets, ACCUMULATE off/on, degenerate sizes), whole output buffer compared
including the elements between rows, with device and with host buffers."""
import numpy as np
import pytest

import conv_testing as C
import uk_testing as T
from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu


def _run_gpu(lib, torch, c, inp, flt, out0, host):
    a = c.args()
    if host:
        got = out0.copy()
        lib.conv_nchwc(inp.ctypes.data, *a["input"], flt.ctypes.data, *a["filter"],
                       got.ctypes.data, *a["output"], *a["dims"])
        return got
    d = [T.DeviceBytes(torch, x) for x in (inp, flt, out0)]
    lib.conv_nchwc(d[0].ptr, *a["input"], d[1].ptr, *a["filter"], d[2].ptr, *a["output"], *a["dims"])
    lib.synchronize()
    return d[2].numpy().view(np.float32)


def _check(lib, torch, oracle, c, ci, host, exact, mfma, atol=1e-4):
    rng = np.random.default_rng(ci)
    inp, flt, out0 = C.buffers(c, rng, exact=exact)
    want = out0.copy()
    C.run(oracle, c, inp, flt, want)
    got = _run_gpu(lib, torch, c, inp, flt, out0, host)
    if exact or not mfma:
        # Small integers: every partial sum is exact, any order gives the same
        # bits. N(0,1) on the scalar kernel: the reference's own order, with a
        # separate multiply and add.
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), c.label()
    else:
        # MFMA order on N(0,1) data: the same sum to f32 rounding. Bound: K
        # products of magnitude |x||w| summed in f32, error <= K * 2^-24 * sum
        # of magnitudes per output; 1e-4 absolute covers K = 432 here with
        # room, and everything the call must not touch is still bit-equal.
        assert np.allclose(got, want, rtol=1e-5, atol=atol), (c.label(), float(np.abs(got - want).max()))
        mask = np.ones(out0.size, bool)
        for nn in range(c.N):
            for oc in range(c.OC_outer):
                for oh in range(c.OH):
                    b = c.offsets[2] + nn * c.out_strides[0] + oc * c.out_strides[1] + oh * c.out_strides[2]
                    mask[b:b + c.OW * c.k0] = False
        assert np.array_equal(got[mask].view(np.uint32), out0[mask].view(np.uint32)), c.label()


@pytest.mark.parametrize("host", [False, True])
@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("mode", [uk.KERNEL_MODE_AUTO, uk.KERNEL_MODE_GENERIC])
def test_conv_reference_test_grid(gpu, oracle, host, exact, mode):
    """The reference test's grid. In AUTO mode the 16x16 tile runs on the MFMA
    kernel, everything else (and everything in GENERIC mode) on the scalar one."""
    lib, torch = gpu
    lib.set_pointer_mode(uk.POINTER_MODE_AUTO)
    lib.set_kernel_mode(mode)
    try:
        for ci, c in enumerate(C.cases(seed=21)):
            mfma = mode == uk.KERNEL_MODE_AUTO and c.k0 == 16 and c.c0 % 16 == 0
            _check(lib, torch, oracle, c, ci, host, exact, mfma)
            early = (c.N == 0 or c.OC_outer == 0 or c.OH == 0 or c.OW == 0 or
                     ((c.IC_outer == 0 or c.FH == 0 or c.FW == 0) and c.flags & C.CONV_ACCUMULATE))
            if not early:
                assert lib.last_kernel_name() == ("conv_nchwc_mfma" if mfma else "conv_nchwc_generic")
    finally:
        lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)


@pytest.mark.parametrize("exact", [True, False])
def test_conv_mfma_wide_shapes(gpu, oracle, exact):
    """Shapes beyond the reference's grid for the MFMA kernel: several panels
    per row (with a partial last one), an odd number of output-channel blocks,
    c0 = 32 and 48, strides 2, loose strides and offsets, ACCUMULATE."""
    lib, torch = gpu
    lib.set_pointer_mode(uk.POINTER_MODE_AUTO)
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    n = 0
    for ci, c in enumerate(C.cases(seed=33, tiles=[(16, 16), (16, 32), (16, 48)],
                                   shapes=C.WIDE_SHAPES)):
        _check(lib, torch, oracle, c, 500 + ci, False, exact, True)
        assert lib.last_kernel_name() == "conv_nchwc_mfma"
        n += 1
    assert n == 24


def test_conv_info_and_fallback_flag(gpu):
    """conv_nchwc.c:139-152,200-218: the info bit names the tile shapes a tuned
    kernel serves; any other shape needs the fallback flag."""
    lib, torch = gpu
    x = torch.zeros(4096, device="cuda")
    info = lib.lib.iree_uk_conv_nchwc_info
    assert info(16, 16, C.CONV_TYPE_F32F32F32, None) == 1
    assert info(16, 32, C.CONV_TYPE_F32F32F32, None) == 1
    assert info(16, 8, C.CONV_TYPE_F32F32F32, None) == 0
    assert info(8, 16, C.CONV_TYPE_F32F32F32, None) == 0
    # 16x16 without the flag: served
    lib.conv_nchwc(x.data_ptr(), 0, 256, 256, 16, x.data_ptr(), 0, 256, 256, 256, x.data_ptr(), 1024,
                   16, 16, 16, 1, 1, 1, 1, 1, 1, 1, 16, 16, 1, 1, C.CONV_TYPE_F32F32F32)
    lib.synchronize()
    with pytest.raises(uk.ContractViolation):
        lib.conv_nchwc(x.data_ptr(), 0, 1, 1, 1, x.data_ptr(), 0, 1, 1, 1, x.data_ptr(), 0, 1, 1, 1,
                       1, 1, 1, 1, 1, 1, 1, 8, 8, 1, 1, C.CONV_TYPE_F32F32F32)


@pytest.mark.parametrize("exact", [True, False])
def test_conv_few_pixels_many_channels_splits_the_input_channels(gpu, oracle, exact):
    """A late layer of an image network at batch 1 (7x7 outputs, 3x3 filter,
    512 -> 512 channels) has fewer output blocks than the device has compute
    units: IC_outer is split over several workgroups per block and a second
    kernel adds the slices up in order. Loose strides, offsets, ACCUMULATE off
    and on; the buffer for the slices shows in iree_uk_amd_workspace_bytes."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    N, OC, OH, OW, IC, FH, FW, k0, c0 = 1, 32, 7, 7, 32, 3, 3, 16, 16
    H, W = OH + FH - 1, OW + FW - 1
    for ci, acc in enumerate((0, 1)):
        in_sh = W * c0 + 16 * ci
        in_sic = H * in_sh + 32 * ci
        f_sfh = FW * c0 * k0
        f_sic = FH * f_sfh + 256 * ci
        out_soh = OW * k0 + 16 * ci
        out_soc = OH * out_soh + 48 * ci
        c = C.ConvCase(N, OC, OH, OW, IC, FH, FW, 1, 1, k0, c0, C.CONV_TYPE_F32F32F32 | (C.CONV_ACCUMULATE if acc else 0),
                       (IC * in_sic, in_sic, in_sh), (IC * f_sic, f_sic, f_sfh), (OC * out_soc, out_soc, out_soh),
                       (4 * ci, 8 * ci, 12 * ci))
        lib.release_workspaces()
        # K = 4608 products per output here, ten times the grid's: two f32
        # summation orders of that many N(0,1) products (sums of magnitude up to
        # a few hundred) differ by a few 1e-4; the exact-data run pins the
        # indexing bit for bit.
        _check(lib, torch, oracle, c, 40 + ci, host=False, exact=exact, mfma=True, atol=2e-3)
        assert lib.last_kernel_name() == "conv_nchwc_mfma"
        assert lib.workspace_bytes() > 0
