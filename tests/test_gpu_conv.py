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


@pytest.mark.parametrize("host", [False, True])
@pytest.mark.parametrize("exact", [True, False])
def test_conv_reference_test_grid(gpu, oracle, host, exact):
    lib, torch = gpu
    lib.set_pointer_mode(uk.POINTER_MODE_AUTO)
    for ci, c in enumerate(C.cases(seed=21)):
        rng = np.random.default_rng(ci)
        inp, flt, out0 = C.buffers(c, rng, exact=exact)
        want = out0.copy()
        C.run(oracle, c, inp, flt, want)
        got = _run_gpu(lib, torch, c, inp, flt, out0, host)
        # N(0,1) inputs too: same accumulation order, separate multiply and add
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), c.label()


def test_conv_without_fallback_flag_is_a_contract_violation(gpu):
    lib, torch = gpu
    x = torch.zeros(64, device="cuda")
    assert lib.lib.iree_uk_conv_nchwc_info(16, 16, C.CONV_TYPE_F32F32F32, None) == 0
    with pytest.raises(uk.ContractViolation):
        lib.conv_nchwc(x.data_ptr(), 0, 1, 1, 1, x.data_ptr(), 0, 1, 1, 1, x.data_ptr(), 0, 1, 1, 1,
                       1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, C.CONV_TYPE_F32F32F32)
