"""The device path launches kernels and nothing else (no allocation, no
memset, no host synchronisation), so a caller may capture calls into a HIP
graph. Each replay is checked against the eager result, with eager work and
synchronisations in between."""
import numpy as np
import pytest

from iree_amd import ukernel as uk


@pytest.mark.gpu
def test_chain_and_fused_calls_replay_from_a_graph(gpu):
    lib, torch = gpu
    M, N, K, M0, N0, K0 = 300, 530, 1024, 16, 16, 16   # ragged: padded tiles, K in whole steps
    M1, N1, K1 = -(-M // M0), -(-N // N0), K // K0
    g = torch.Generator(device="cuda"); g.manual_seed(21)
    a = torch.randint(-128, 128, (M, K), generator=g, device="cuda", dtype=torch.int8)
    bt = torch.randint(-128, 128, (N, K), generator=g, device="cuda", dtype=torch.int8)
    rs = torch.rand(M, generator=g, device="cuda") + 0.5
    cs = torch.rand(N, generator=g, device="cuda") + 0.5
    lhs4 = torch.zeros(M1 * K1 * M0 * K0, device="cuda", dtype=torch.int8)
    rhs4 = torch.zeros(N1 * K1 * N0 * K0, device="cuda", dtype=torch.int8)
    out4 = torch.zeros(M1 * N1 * M0 * N0, device="cuda", dtype=torch.int32)
    out = torch.zeros(M, N, device="cuda", dtype=torch.int32)
    y = torch.zeros(M, N, device="cuda", dtype=torch.float32)
    flags = uk.MMT4D_TYPE_S8S8S32

    def step():
        lib.pack(a.data_ptr(), 0, K, 1, lhs4.data_ptr(), 0, K1 * M0 * K0, M0 * K0, M, K, M1, K1, M0, K0,
                 0, uk.PACK_TYPE_I8I8)
        lib.pack(bt.data_ptr(), 0, K, 1, rhs4.data_ptr(), 0, K1 * N0 * K0, N0 * K0, N, K, N1, K1, N0, K0,
                 0, uk.PACK_TYPE_I8I8)
        lib.mmt4d(lhs4.data_ptr(), 0, K1 * M0 * K0, rhs4.data_ptr(), 0, K1 * N0 * K0, out4.data_ptr(), 0,
                  N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags)
        lib.unpack(out4.data_ptr(), 0, N1 * M0 * N0, M0 * N0, out.data_ptr(), 0, N, 1, M1, N1, M0, N0,
                   M, N, uk.UNPACK_TYPE_I32I32)
        lib.mmt4d_dequant_unpack(lhs4.data_ptr(), 0, K1 * M0 * K0, rhs4.data_ptr(), 0, K1 * N0 * K0,
                                 None, 0, 0, y.data_ptr(), 0, N, M, N, rs.data_ptr(), cs.data_ptr(),
                                 M1, N1, K1, M0, N0, K0, flags)

    stream = torch.cuda.Stream()
    lib.set_pointer_mode(uk.POINTER_MODE_DEVICE)   # no pointer queries while capturing
    lib.set_stream(stream.cuda_stream)
    try:
        with torch.cuda.stream(stream):
            step()
        stream.synchronize()
        want = (a.cpu().to(torch.int64) @ bt.cpu().to(torch.int64).T).to(torch.int32)
        assert torch.equal(out.cpu(), want)
        want_y = (want.float() * rs.cpu()[:, None]) * cs.cpu()[None, :]
        assert torch.equal(y.cpu(), want_y)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step()
        torch.cuda.synchronize()
        for rep in range(3):
            for t in (lhs4, rhs4, out4, out, y):
                t.zero_()                       # eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.cpu(), want), rep
            assert torch.equal(y.cpu(), want_y), rep
    finally:
        lib.set_stream(None)
        lib.set_pointer_mode(uk.POINTER_MODE_AUTO)


@pytest.mark.gpu
def test_k_split_call_under_capture_takes_no_library_workspace(gpu):
    """A decode-shaped mmt4d (few rows, long K: eagerly the thin kernel splits K
    over workgroups through a workspace the library owns per thread and stream)
    captured into a graph: the capturing stream is never handed such a
    workspace - the graph would outlive it and share it with eager calls - so
    the captured call runs without the split. Replays, with eager K-split calls
    on the same thread and stream in between, equal the exact integer product."""
    lib, torch = gpu
    Mrows, N, K, M0, N0, K0 = 16, 1024, 14336, 16, 16, 16
    M1, N1, K1 = 1, N // N0, K // K0
    g = torch.Generator(device="cuda"); g.manual_seed(23)
    lhs = torch.randint(-128, 128, (M1 * K1 * M0 * K0,), generator=g, device="cuda", dtype=torch.int8)
    rhs = torch.randint(-128, 128, (N1 * K1 * N0 * K0,), generator=g, device="cuda", dtype=torch.int8)
    out_eager = torch.zeros(M1 * N1 * M0 * N0, device="cuda", dtype=torch.int32)
    out_graph = torch.zeros_like(out_eager)
    a = lhs.view(M1, K1, M0, K0).permute(0, 2, 1, 3).reshape(M0, K).cpu().to(torch.int64)
    b = rhs.view(N1, K1, N0, K0).permute(0, 2, 1, 3).reshape(N, K).cpu().to(torch.int64)
    want = (a @ b.T).to(torch.int32).view(M1, M0, N1, N0).permute(0, 2, 1, 3).reshape(-1)

    def call(out):
        lib.mmt4d(lhs.data_ptr(), 0, K1 * M0 * K0, rhs.data_ptr(), 0, K1 * N0 * K0, out.data_ptr(), 0,
                  N1 * M0 * N0, M1, N1, K1, M0, N0, K0, uk.MMT4D_TYPE_S8S8S32)

    stream = torch.cuda.Stream()
    lib.set_pointer_mode(uk.POINTER_MODE_DEVICE)
    lib.set_stream(stream.cuda_stream)
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_k_slices(0)
    try:
        with torch.cuda.stream(stream):
            call(out_eager)                    # creates this thread's workspace for the stream
        stream.synchronize()
        assert lib.last_k_slices() > 1, lib.last_kernel_name()
        assert torch.equal(out_eager.cpu(), want)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            call(out_graph)
            slices_under_capture = lib.last_k_slices()
        torch.cuda.synchronize()
        assert slices_under_capture == 1
        for rep in range(3):
            out_graph.zero_()
            out_eager.zero_()
            with torch.cuda.stream(stream):
                call(out_eager)                # an eager K-split call between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_graph.cpu(), want), rep
            assert torch.equal(out_eager.cpu(), want), rep
    finally:
        lib.set_stream(None)
        lib.set_pointer_mode(uk.POINTER_MODE_AUTO)
