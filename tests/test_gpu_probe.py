"""The lane mapping of ds_read_b64_tr_b16, which the mmt4d kernels' fragment
reads for 2-byte tile rows (the reference's x86 tile 16x16x2 of s8,
arch/x86_64/mmt4d_x86_64_tiles.inl:10-75) rest on: within a block of 16
lanes, lane i receives as element j the element i % 4 of the eight bytes that
lane 4 j + i / 4 of the same block addressed."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _model(lane_index):
    want = np.zeros((64, 4), np.int16)
    for lane in range(64):
        block, i = lane // 16, lane % 16
        for j in range(4):
            src = block * 16 + 4 * j + i // 4
            want[lane, j] = lane_index[src] + i % 4
    return want


@pytest.mark.parametrize("pattern", ["contiguous", "fragment", "random"])
def test_ds_read_tr16_lane_mapping(gpu, pattern):
    lib, torch = gpu
    rng = np.random.default_rng(5)
    if pattern == "contiguous":
        idx = 4 * np.arange(64)
    elif pattern == "fragment":
        # the addresses of the kernels' fragment read: lane (q, r) addresses rows
        # 4 (r % 4) .. + 3 of K-tile 4 q + r / 4 in a [K-tile][16 rows][2 bytes] image
        lane = np.arange(64)
        q, r = lane // 16, lane % 16
        idx = (4 * q + r // 4) * 16 + (r % 4) * 4
    else:
        idx = 4 * rng.integers(0, 4096, 64)
    d_idx = torch.from_numpy(idx.astype(np.int32)).to("cuda")
    d_out = torch.zeros(256, dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()
    lib.probe_ds_read_tr16(d_idx.data_ptr(), d_out.data_ptr(), 16384, torch.cuda.current_stream().cuda_stream)
    got = d_out.cpu().numpy().reshape(64, 4)
    assert np.array_equal(got, _model(idx)), (pattern, got[:8], _model(idx)[:8])
    if pattern == "fragment":
        # what the kernel needs from it: lane (q, r) ends up with row r of K-tiles 4 q .. 4 q + 3
        lane = np.arange(64)
        q, r = lane // 16, lane % 16
        for j in range(4):
            assert np.array_equal(got[:, j], (4 * q + j) * 16 + r)
