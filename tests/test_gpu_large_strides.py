"""Strides beyond 2 GiB: the fast kernels index inside a workgroup's share with
32-bit offsets and must hand such calls to the kernels with 64-bit indexing
(runtime/src/iree/builtins/ukernel/mmt4d.c:70-100 and pack.c:254-313 do all of
their pointer arithmetic in iree_uk_index_t = int64). Operands live on the GPU
only; expectations come from the small dense pieces."""
import numpy as np
import pytest

from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu


def test_mmt4d_panel_stride_above_2gib(gpu):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, K1, M0, N0, K0 = 2, 3, 4, 16, 16, 16
    panel = K1 * M0 * K0
    lhs_stride = (1 << 31) + 4096                      # elements = bytes (s8)
    g = torch.Generator(device="cuda"); g.manual_seed(31)
    lhs = torch.zeros(lhs_stride * (M1 - 1) + panel, device="cuda", dtype=torch.int8)
    panels = torch.randint(-128, 128, (M1, panel), generator=g, device="cuda", dtype=torch.int8)
    for i in range(M1):
        lhs[i * lhs_stride:i * lhs_stride + panel] = panels[i]
    rhs = torch.randint(-128, 128, (N1, K1, N0, K0), generator=g, device="cuda", dtype=torch.int8)
    out = torch.zeros(M1, N1, M0, N0, device="cuda", dtype=torch.int32)
    lib.mmt4d(lhs.data_ptr(), 0, lhs_stride, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32 | 0x200)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_generic"
    a = panels.view(M1, K1, M0, K0).permute(0, 2, 1, 3).reshape(M1 * M0, K1 * K0).cpu().to(torch.int64)
    b = rhs.permute(0, 2, 1, 3).reshape(N1 * N0, K1 * K0).cpu().to(torch.int64)
    want = (a @ b.T).reshape(M1, M0, N1, N0).permute(0, 2, 1, 3)
    assert torch.equal(out.cpu().to(torch.int64), want)


def test_pack_and_unpack_row_pitch_whose_block_span_exceeds_2gib(gpu):
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    rows, cols, t0, t1 = 20, 70, 16, 16
    pitch = 1 << 28                                     # elements = bytes (s8): 16 rows span 4 GiB
    g = torch.Generator(device="cuda"); g.manual_seed(32)
    src = torch.zeros(pitch * (rows - 1) + cols, device="cuda", dtype=torch.int8)
    dense = torch.randint(-128, 128, (rows, cols), generator=g, device="cuda", dtype=torch.int8)
    for r in range(rows):
        src[r * pitch:r * pitch + cols] = dense[r]
    o0, o1 = -(-rows // t0), -(-cols // t1)
    packed = torch.zeros(o0 * o1 * t0 * t1, device="cuda", dtype=torch.int8)
    lib.pack(src.data_ptr(), 0, pitch, 1, packed.data_ptr(), 0, o1 * t0 * t1, t0 * t1, rows, cols,
             o0, o1, t0, t1, 0x7F, uk.PACK_TYPE_I8I8)
    lib.synchronize()
    padded = torch.full((o0 * t0, o1 * t1), 0x7F, dtype=torch.int8)
    padded[:rows, :cols] = dense.cpu()
    want = padded.view(o0, t0, o1, t1).permute(0, 2, 1, 3).reshape(-1)
    assert torch.equal(packed.cpu(), want)
    # and back, as 4-byte elements, into rows a 2^28-element pitch apart
    rows4, cols4 = 20, 24
    tiled = torch.randint(-1000, 1000, (2, 2, 16, 16), generator=g, device="cuda", dtype=torch.int32)
    pitch4 = 1 << 28                                    # int32 elements: 1 GiB per row
    dst = torch.zeros(pitch4 * (rows4 - 1) + cols4, device="cuda", dtype=torch.int32)
    lib.unpack(tiled.data_ptr(), 0, 2 * 256, 256, dst.data_ptr(), 0, pitch4, 1, 2, 2, 16, 16,
               rows4, cols4, uk.UNPACK_TYPE_I32I32)
    lib.synchronize()
    want4 = tiled.permute(0, 2, 1, 3).reshape(32, 32)[:rows4, :cols4].cpu()
    got4 = torch.stack([dst[r * pitch4:r * pitch4 + cols4] for r in range(rows4)]).cpu()
    assert torch.equal(got4, want4)


def test_mmt4d_negative_panel_stride_takes_the_signed_64_bit_kernel(gpu):
    """A negative outer stride walks the panels backwards (mmt4d.c:70-100 does
    signed index arithmetic and, unlike pack.c:69-71, asserts no sign): equal
    to the forward call with the row panels reversed."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, K1, M0, N0, K0 = 5, 3, 8, 16, 16, 16
    panel = K1 * M0 * K0
    g = torch.Generator(device="cuda"); g.manual_seed(33)
    lhs = torch.randint(-128, 128, (M1, panel), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1, K1 * N0 * K0), generator=g, device="cuda", dtype=torch.int8)
    fwd = torch.zeros(M1, N1 * M0 * N0, device="cuda", dtype=torch.int32)
    lib.mmt4d(lhs.data_ptr(), 0, panel, rhs.data_ptr(), 0, K1 * N0 * K0, fwd.data_ptr(), 0, N1 * M0 * N0,
              M1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32 | 0x200)
    assert lib.last_kernel_name().startswith("mmt4d_mfma")
    bwd = torch.zeros_like(fwd)
    lib.mmt4d(lhs.data_ptr(), (M1 - 1) * panel, -panel, rhs.data_ptr(), 0, K1 * N0 * K0, bwd.data_ptr(), 0,
              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32 | 0x200)
    lib.synchronize()
    assert lib.last_kernel_name() == "mmt4d_generic"
    assert torch.equal(bwd, fwd.flip(0))
