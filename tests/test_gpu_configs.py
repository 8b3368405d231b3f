"""The benchmark configurations at their FULL sizes, through the C-ABI, against
the CPU oracle.

A full-size output cannot be recomputed on the CPU in test time, so -- as the
reference's own end-to-end benchmark does when it validates a run
(runtime/src/iree/builtins/ukernel/tools/e2e_matmul_benchmark.c:337-358 checks
the result of the timed chain against an independent computation) -- mmt4d
results are checked on a sample: at least 64 output tiles drawn at random, each
over all of K, plus every tile of the last tile row and column when the
problem is ragged, plus the four corners. Each sampled tile is one oracle call
with M = N = 1 on the panels of that tile. pack / unpack results are compared
in full with their numpy formulation (pad + reshape + transpose) and round
trips. The 1024^3 configuration is compared in full.

Bars: bit-exact for s8 and for pack / unpack; max|gpu - ref| / max|ref| over
the sampled elements <= 1e-2 for f16 / bf16 and <= 2e-2 for f8 against the
f32-accumulating oracle. The first mismatch stops the test.
"""
import numpy as np
import pytest

from iree_amd import ukernel as uk

pytestmark = pytest.mark.gpu

ES = {"s8": 1, "f8": 1, "f16": 2, "bf16": 2}
TYPE = {"s8": uk.MMT4D_TYPE_S8S8S32, "f16": uk.MMT4D_TYPE_F16F16F32,
        "bf16": uk.MMT4D_TYPE_BF16BF16F32, "f8": uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32}
TOL = {"f16": 1e-2, "bf16": 1e-2, "f8": 2e-2}


@pytest.fixture()
def runner(gpu):
    lib, torch = gpu
    from iree_amd.runner import Runner
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    r = Runner(seed=0)
    yield r
    r.close()
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    torch.cuda.empty_cache()


def _host(t):
    import torch
    return t.contiguous().view(torch.uint8).cpu().numpy()


def sample_tiles(M1, N1, n_random, rng, ragged=False):
    tiles = {(0, 0), (0, N1 - 1), (M1 - 1, 0), (M1 - 1, N1 - 1)}
    if ragged:
        tiles |= {(M1 - 1, n) for n in range(N1)} | {(m, N1 - 1) for m in range(M1)}
    while len(tiles) < n_random + 4 + (M1 + N1 - 1 if ragged else 0):
        tiles.add((int(rng.integers(M1)), int(rng.integers(N1))))
    return sorted(tiles)


def check_mmt4d_tiles(oracle, dtype, lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0, tiles,
                      accumulate_from=None):
    """Compares out4 (device tensor, [M1][N1][M0][N0] 4-byte elements) with the
    oracle on the given (m, n) tiles. lhs4 / rhs4 are the packed device
    operands. Returns the error measure (0.0 for a bit-exact s8 pass)."""
    es = ES[dtype]
    lhs = _host(lhs4).reshape(M1, K1 * M0 * K0 * es)
    rhs = _host(rhs4).reshape(N1, K1 * N0 * K0 * es)
    got_all = _host(out4).view(np.int32 if dtype == "s8" else np.float32).reshape(M1, N1, M0 * N0)
    flags = TYPE[dtype] | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    out_dt = np.int32 if dtype == "s8" else np.float32
    view = {1: np.uint8, 2: np.uint16}[es]
    max_err, max_ref = 0.0, 0.0
    for (m, n) in tiles:
        want = np.zeros(M0 * N0, out_dt)
        if accumulate_from is not None:
            want[:] = accumulate_from.reshape(M1, N1, M0 * N0)[m, n]
        f = flags | (uk.MMT4D_ACCUMULATE if accumulate_from is not None else 0)
        oracle.mmt4d(lhs[m].view(view), 0, 0, rhs[n].view(view), 0, 0, want, 0, 0, 1, 1, K1,
                     M0, N0, K0, f)
        got = got_all[m, n]
        if dtype == "s8":
            assert np.array_equal(got, want), f"tile ({m}, {n}) differs from the oracle"
        else:
            assert np.isfinite(got).all() and np.isfinite(want).all(), f"non-finite value in tile ({m}, {n})"
            max_err = max(max_err, float(np.abs(got - want).max()))
            max_ref = max(max_ref, float(np.abs(want).max()))
    if dtype == "s8":
        return 0.0
    assert max_ref > 0
    err = max_err / max_ref
    assert err <= TOL[dtype], f"max|gpu-ref|/max|ref| = {err:.3e} > {TOL[dtype]}"
    return err


def pack_identity(x, tile0, tile1, pad, transpose_outer=False):
    """numpy formulation of iree_uk_pack without TRANSPOSE_INNER: pad to whole
    tiles, split both dims, bring the tile dims innermost."""
    rows, cols = x.shape
    o0, o1 = -(-rows // tile0), -(-cols // tile1)
    p = np.full((o0 * tile0, o1 * tile1), pad, dtype=x.dtype)
    p[:rows, :cols] = x
    p = p.reshape(o0, tile0, o1, tile1)
    return np.ascontiguousarray(p.transpose(2, 0, 1, 3) if transpose_outer else p.transpose(0, 2, 1, 3))


def run_ops(r, wl, names=None):
    torch = r.torch
    # The ops launch on the runner's stream; anything the test itself enqueued
    # with torch (fills of the outputs) sits on torch's stream: finish it first.
    torch.cuda.synchronize()
    with torch.cuda.stream(r.stream):
        for op in wl.ops:
            if names is None or op.name in names:
                op.launch()
                if not op.external:
                    op.kernel = r.lib.last_kernel_name()
    r.stream.synchronize()


def test_c1_s8_1024_tiles_16x16x2_full_compare(runner, oracle):
    wl = runner.workload("s8_mmt4d_1024_k2")
    run_ops(runner, wl)
    k = wl.keep
    M1, N1, K1, M0, N0, K0 = (k[x] for x in ("M1", "N1", "K1", "M0", "N0", "K0"))
    assert wl.ops[0].kernel.startswith("mmt4d_mfma"), wl.ops[0].kernel
    lhs, rhs = _host(k["lhs4"]).view(np.int8), _host(k["rhs4"]).view(np.int8)
    want = np.zeros(M1 * N1 * M0 * N0, np.int32)
    oracle.mmt4d(lhs, 0, K1 * M0 * K0, rhs, 0, K1 * N0 * K0, want, 0, N1 * M0 * N0, M1, N1, K1,
                 M0, N0, K0, uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
    assert np.array_equal(_host(k["out4"]).view(np.int32), want)


@pytest.mark.parametrize("name", ["c2_f16_chain_4096", "c2_f16_chain_ragged"])
def test_c2_f16_chain_at_size(runner, oracle, name):
    wl = runner.workload(name)
    run_ops(runner, wl)
    k = wl.keep
    M, N, K, M0, N0, K0 = (k[x] for x in ("M", "N", "K", "M0", "N0", "K0"))
    M1, N1, K1 = -(-M // M0), -(-N // N0), K // K0
    a = _host(k["a"]).view(np.uint16).reshape(M, K)
    bt = _host(k["bt"]).view(np.uint16).reshape(N, K)
    # pack: the whole packed buffers against the numpy formulation (pad 0)
    assert np.array_equal(_host(k["lhs4"]).view(np.uint16), pack_identity(a, M0, K0, 0).reshape(-1))
    assert np.array_equal(_host(k["rhs4"]).view(np.uint16), pack_identity(bt, N0, K0, 0).reshape(-1))
    # mmt4d: sampled tiles (+ the whole ragged edge) against the oracle
    rng = np.random.default_rng(2)
    tiles = sample_tiles(M1, N1, 64, rng, ragged=name.endswith("ragged"))
    check_mmt4d_tiles(oracle, "f16", k["lhs4"], k["rhs4"], k["out4"], M1, N1, K1, M0, N0, K0, tiles)
    # unpack: the whole matrix against the tiled result it was made from
    out4 = _host(k["out4"]).view(np.float32).reshape(M1, N1, M0, N0)
    want = out4.transpose(0, 2, 1, 3).reshape(M1 * M0, N1 * N0)[:M, :N]
    assert np.array_equal(_host(k["out"]).view(np.float32).reshape(M, N), want)


def test_c4_f8_prefill_at_size(runner, oracle):
    wl = runner.workload("c4_f8_prefill")
    run_ops(runner, wl)
    k = wl.keep
    M, N, K, M1, N1, K1, M0, N0, K0 = (k[x] for x in ("M", "N", "K", "M1", "N1", "K1", "M0", "N0", "K0"))
    assert np.array_equal(_host(k["lhs4"]), pack_identity(_host(k["a"]).reshape(M, K), M0, K0, 0).reshape(-1))
    assert np.array_equal(_host(k["rhs4"]), pack_identity(_host(k["bt"]).reshape(N, K), N0, K0, 0).reshape(-1))
    tiles = sample_tiles(M1, N1, 64, np.random.default_rng(4))
    check_mmt4d_tiles(oracle, "f8", k["lhs4"], k["rhs4"], k["out4"], M1, N1, K1, M0, N0, K0, tiles)


@pytest.mark.parametrize("name,dtype", [("bf16_mmt4d_8192_k2", "bf16"), ("bf16_mmt4d_8192_k8", "bf16"),
                                        ("f8_mmt4d_8192_k32", "f8")])
def test_c5_float_mmt4d_8192_sampled_tiles(runner, oracle, name, dtype):
    wl = runner.workload(name)
    run_ops(runner, wl)
    k = wl.keep
    M1, N1, K1, M0, N0, K0 = (k[x] for x in ("M1", "N1", "K1", "M0", "N0", "K0"))
    assert wl.ops[0].kernel.startswith("mmt4d_mfma"), wl.ops[0].kernel
    tiles = sample_tiles(M1, N1, 64, np.random.default_rng(5))
    check_mmt4d_tiles(oracle, dtype, k["lhs4"], k["rhs4"], k["out4"], M1, N1, K1, M0, N0, K0, tiles)


# The s8 8192^3 target: the reference's own x86 tile (16x16x2) and an
# MFMA-friendly K0, bit-exact on the sampled tiles; the K0 = 16 case also under
# every big workgroup shape (1 = 256x256, 8 = 128x512, 9 / 10 = persistent,
# 16 / 17 = the LDS-direct pipeline in the 256x256 / 128x512 shape).
@pytest.mark.parametrize("name,variant", [("s8_mmt4d_8192_k2", 0), ("s8_mmt4d_8192_k16", 0),
                                          ("s8_mmt4d_8192_k16", 1), ("s8_mmt4d_8192_k16", 8),
                                          ("s8_mmt4d_8192_k16", 9), ("s8_mmt4d_8192_k16", 10),
                                          ("s8_mmt4d_8192_k16", 16), ("s8_mmt4d_8192_k16", 17),
                                          ("s8_mmt4d_8192_k64", 0)])
def test_target_s8_mmt4d_8192_bit_exact_on_sampled_tiles(runner, oracle, name, variant):
    wl = runner.workload(name)
    k = wl.keep
    k["out4"].fill_(-1)
    runner.lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
    try:
        run_ops(runner, wl)
    finally:
        runner.lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    M1, N1, K1, M0, N0, K0 = (k[x] for x in ("M1", "N1", "K1", "M0", "N0", "K0"))
    assert wl.ops[0].kernel.startswith("mmt4d_mfma"), wl.ops[0].kernel
    tiles = sample_tiles(M1, N1, 96, np.random.default_rng(8 + variant))
    check_mmt4d_tiles(oracle, "s8", k["lhs4"], k["rhs4"], k["out4"], M1, N1, K1, M0, N0, K0, tiles)
    # Every workgroup block stored something: no element kept the fill value
    # in all four bytes on a uniform-random problem (probability ~ 2^-32 each).
    import torch
    assert int((k["out4"].view(M1, N1, M0 * N0) == -1).all(dim=2).sum().item()) == 0


@pytest.mark.parametrize("name", ["c5_pack_f32_12288x12289", "c5_pack_f32_12289x12288"])
def test_c5_pack_unpack_stress_at_size(runner, name):
    wl = runner.workload(name)
    k = wl.keep
    k["packed"].fill_(7.0)
    k["back"].fill_(7.0)
    run_ops(runner, wl)
    rows, cols = k["rows"], k["cols"]
    x = _host(k["x"]).view(np.uint32).reshape(rows, cols)
    want = pack_identity(x, 16, 1, np.uint32(0xBF800000), transpose_outer=True).reshape(-1)
    got = _host(k["packed"]).view(np.uint32)
    assert got.shape == want.shape
    assert np.array_equal(got, want), "packed buffer differs from pad + reshape + transpose"
    del want, got
    assert np.array_equal(_host(k["back"]).view(np.uint32).reshape(rows, cols), x), "round trip"


@pytest.mark.parametrize("rows,cols,es,t0,t1,pitch_slack", [(8190, 8200, 4, 16, 16, 0),     # f32, 256 MB, ragged
                                                            (8192, 8192, 4, 16, 16, 1),     # loose pitch, rows only 4-byte aligned
                                                            (12272, 8192, 1, 16, 32, 0)])   # f8/s8 rows, ragged
def test_row_granule_pack_unpack_in_64k_blocks_at_size(gpu, rows, cols, es, t0, t1, pitch_slack):
    """Untransposed pack / unpack of large matrices (whole tile rows move as
    16-byte granules, 64 KB blocks per workgroup): the packed buffer equals
    pad + reshape + transpose of the source, padding included, and unpack
    restores the matrix and leaves the pitch gap alone."""
    lib, torch = gpu
    ty = {1: uk.PACK_TYPE_I8I8, 4: uk.PACK_TYPE_F32F32}[es]
    dt = {1: torch.uint8, 4: torch.int32}[es]
    npdt = {1: np.uint8, 4: np.uint32}[es]
    pitch = cols + pitch_slack
    hi = 256 if es == 1 else 2 ** 31 - 1
    x = torch.randint(0, hi, (rows, pitch), dtype=dt, device="cuda")
    o0, o1 = -(-rows // t0), -(-cols // t1)
    packed = torch.full((o0 * o1 * t0 * t1,), 3, dtype=dt, device="cuda")
    back = torch.full((rows, pitch), 5, dtype=dt, device="cuda")
    pad = 0x5A if es == 1 else 0x5A5A5A5A
    torch.cuda.synchronize()
    lib.pack(x.data_ptr(), 0, pitch, 1, packed.data_ptr(), 0, o1 * t0 * t1, t0 * t1, rows, cols,
             o0, o1, t0, t1, pad, ty)
    assert lib.last_kernel_name() == "pack_stream"
    if es != 1:     # unpack has no 1-byte type (exported_bits.h:73-79)
        lib.unpack(packed.data_ptr(), 0, o1 * t0 * t1, t0 * t1, back.data_ptr(), 0, pitch, 1,
                   o0, o1, t0, t1, rows, cols, uk.UNPACK_TYPE_F32F32)
        assert lib.last_kernel_name() == "unpack_stream"
    lib.synchronize()
    xh = x.cpu().numpy().view(npdt)[:, :cols]
    want = pack_identity(xh, t0, t1, npdt(pad)).reshape(-1)
    assert np.array_equal(packed.cpu().numpy().view(npdt), want), "packed buffer"
    if es != 1:
        bh = back.cpu().numpy().view(npdt)
        assert np.array_equal(bh[:, :cols], xh), "round trip"
        assert (bh[:, cols:] == 5).all(), "pitch gap written"
