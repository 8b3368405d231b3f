#!/usr/bin/env python3
"""Benchmark of the gfx950 pack / mmt4d / unpack ukernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]
                    [--no-extra] [--no-cpu]
    python bench.py --sweep WORKLOAD     (T(K) table of a square mmt4d workload)

A step is one pass of the workload's whole chain over one batch of seeded
synthetic tensors that are already resident in HBM. The default workload is
the f16 pack -> mmt4d -> unpack chain at M=N=K=4096 with 16x16x16 tiles. One
JSON line is printed; `roofline` describes the dominant kernel (mmt4d),
`cpu_baseline` the same chain on the host cores, `extra` carries the other
benchmark configurations (kernel-level event timings, each with its own CPU
baseline), `measured_mfma_only_TOPS` and `measured_copy_GBps` the ceilings
measured in this run, `host` the cores the CPU baselines saw and used, and
`targets`, the last object of the line, one compact row per target workload:
kernel, time, fraction of the published peak and of the measured ceiling, and
the parity check made on the result that was just timed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

EXTRA_WORKLOADS = [
    "s8_mmt4d_8192_k2", "s8_mmt4d_8192_k16", "s8_mmt4d_8192_k16_zeros", "s8_mmt4d_8192_k64",
    "s8_mmt4d_1024_k2",
    "c2_f16_chain_ragged", "c2_f16_fused_4096", "c2_f16_fused_ragged", "c3_s8_decode",
    "c3_s8_decode_fused", "c3_s8_decode_down", "c3_s8_decode_cold", "c3_s8_decode_fused_cold",
    "c4_f8_prefill",
    "bf16_mmt4d_8192_k2", "bf16_mmt4d_8192_k8", "f8_mmt4d_8192_k32", "f32_mmt4d_4096_k1",
    "f32_mmt4d_4096_k4", "s16_mmt4d_4096_k2",
    "c5_pack_f32_12288x12289", "c5_pack_f32_12289x12288", "pack_operand_forms",
    "conv_nchwc_f32_n16_56x56_c256_k256_3x3",
]


# HBM-bound kernels that move this much or more are also timed with the
# memory-side cache emptied before every launch.
COLD_FROM_BYTES = 32 << 20


def recorded_traffic(workload: str, op: str, kernel: str):
    """(bytes, source): HBM-side bytes per launch of the dominant kernel from
    the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary of this
    workload (counters cannot be read from inside the process), and the file
    it was read from. (None, reason) when there is no summary or when the
    summary was recorded for another kernel than the one that ran now."""
    if op != "mmt4d":
        return None, "no counter summary for this op"
    rel = os.path.join("profiles", f"{workload}_hbm_traffic.txt")
    value, recorded_kernel = None, None
    try:
        with open(os.path.join(ROOT, rel)) as f:
            for line in f:
                if line.startswith("mmt4d_traffic_bytes_per_launch:"):
                    value = int(line.split(":")[1])
                if line.startswith("mmt4d_kernel:"):
                    recorded_kernel = line.split(":")[1].strip()
    except OSError:
        return None, f"{rel} not found"
    if value is None:
        return None, f"{rel} holds no figure"
    if recorded_kernel != kernel:
        return None, f"{rel} was recorded for kernel {recorded_kernel!r}, this run used {kernel!r}"
    return value, f"{rel} (recorded rocprofv3 --pmc run of this command, not measured in this run)"


CPU_THREAD_CAP = 16   # a one-GPU box gives a job 16 cores' worth of CPU whatever nproc says


def cpu_info() -> dict:
    """Host cores as seen and threads as used by the CPU baselines."""
    nproc = os.cpu_count() or 1
    try:
        affinity = len(os.sched_getaffinity(0))
    except AttributeError:
        affinity = nproc
    n = affinity
    omp = os.environ.get("OMP_NUM_THREADS", "")
    if omp.isdigit():
        n = min(n, int(omp))
    return {"nproc": nproc, "affinity": affinity, "OMP_NUM_THREADS": omp or None,
            "thread_cap": CPU_THREAD_CAP, "threads_used": max(1, min(n, CPU_THREAD_CAP))}


def cpu_threads() -> int:
    return cpu_info()["threads_used"]


def cpu_baseline_c2(keep: dict, target_seconds: float = 12.0) -> dict:
    """The f16 chain on the host: the compiled reference C ukernels when
    oracle/_ref holds them (kind "reference"), else the C restatement (kind
    "port"). pack of both operands runs in full; mmt4d and unpack run on a slab
    of M tile-rows sized for about `target_seconds`, split over threads through
    the offset/stride parameters, and are extrapolated to the whole problem."""
    import numpy as np
    from oracle import uk_oracle
    from iree_amd import ukernel as uk

    kind = "reference" if uk_oracle.Checker.reference_available() else "port"
    chk = uk_oracle.Checker("reference" if kind == "reference" else "oracle")
    chk.use_host_cpu_features(True)
    T = cpu_threads()
    M, N, K = keep["M"], keep["N"], keep["K"]
    M0, N0, K0 = keep["M0"], keep["N0"], keep["K0"]
    M1, N1, K1 = -(-M // M0), -(-N // N0), K // K0
    a = keep["a"].cpu().numpy().view(np.uint16)
    bt = keep["bt"].cpu().numpy().view(np.uint16)
    lhs4 = np.zeros(M1 * K1 * M0 * K0, np.uint16)
    rhs4 = np.zeros(N1 * K1 * N0 * K0, np.uint16)
    t0 = time.perf_counter()
    chk.pack(a, 0, K, 1, lhs4, 0, K1 * M0 * K0, M0 * K0, M, K, M1, K1, M0, K0, 0, uk.PACK_TYPE_F16F16)
    chk.pack(bt, 0, K, 1, rhs4, 0, K1 * N0 * K0, N0 * K0, N, K, N1, K1, N0, K0, 0, uk.PACK_TYPE_F16F16)
    t_pack = time.perf_counter() - t0
    flags = uk.MMT4D_TYPE_F16F16F32 | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    # Calibrate on one tile-row per thread, then size the slab.
    out4 = np.zeros(M1 * N1 * M0 * N0, np.float32)
    t0 = time.perf_counter()
    chk.mmt4d_threaded(T, lhs4, K1 * M0 * K0, rhs4, K1 * N0 * K0, out4, N1 * M0 * N0,
                       T, N1, K1, M0, N0, K0, flags)
    t_cal = time.perf_counter() - t0
    slab = int(max(T, min(M1, T * round(target_seconds / max(t_cal, 1e-3)))))
    slab -= slab % T
    t0 = time.perf_counter()
    chk.mmt4d_threaded(T, lhs4, K1 * M0 * K0, rhs4, K1 * N0 * K0, out4, N1 * M0 * N0,
                       slab, N1, K1, M0, N0, K0, flags)
    t_mm = time.perf_counter() - t0
    out = np.zeros(M * N, np.float32)
    rows = min(M, slab * M0)
    t0 = time.perf_counter()
    chk.unpack(out4, 0, N1 * M0 * N0, M0 * N0, out, 0, N, 1, slab, N1, M0, N0, rows, N,
               uk.UNPACK_TYPE_F32F32)
    t_un = time.perf_counter() - t0
    total = t_pack + (t_mm + t_un) * (M1 / slab)
    return {
        "value": round(2.0 * M * N * K / total / 1e12, 6), "unit": "TFLOP/s", "cores": T,
        "kind": kind,
        "sample": (f"pack of both operands in full (1 thread, {t_pack:.2f} s); mmt4d on "
                   f"{slab}/{M1} M tile-rows over {T} threads ({t_mm:.2f} s, generic f16 tile "
                   f"function: no x86 tile exists for 16x16x16) and unpack of those rows "
                   f"({t_un:.2f} s), extrapolated x{M1 / slab:.1f}"),
    }, out4, slab


def _host_bytes(t):
    """A device tensor as a flat numpy byte view on the host."""
    import torch
    return t.contiguous().view(torch.uint8).cpu().numpy()


def _mmt4d_type_flag(dtype: str, uk):
    return {"s8": uk.MMT4D_TYPE_S8S8S32, "f16": uk.MMT4D_TYPE_F16F16F32,
            "bf16": uk.MMT4D_TYPE_BF16BF16F32, "f32": uk.MMT4D_TYPE_F32F32F32,
            "f8": uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, "s16": uk.MMT4D_TYPE_S16S16S32}[dtype]


def cpu_baseline_extra(wl, target_seconds: float = 3.0):
    """The CPU path beside an `extra` workload, on a bounded sample: the
    compiled reference with the host's ISA paths enabled where it has the type
    (kind "reference"; s8 16x16x2 and bf16 16x16x2 then run its AVX-512
    VNNI / BF16 tiles), the C restatement for f8 (kind "port"). mmt4d runs on
    a slab of tile rows (or columns when M is one tile) over all threads, sized
    from a calibration run and extrapolated; pack / unpack run single-threaded
    on a slab of rows. None for workloads it does not cover."""
    import numpy as np
    from oracle import uk_oracle
    from iree_amd import ukernel as uk

    keep = wl.keep
    T = cpu_threads()
    have_ref = uk_oracle.Checker.reference_available()
    if wl.name.startswith("c5_pack"):
        chk = uk_oracle.Checker("reference" if have_ref else "oracle")
        chk.use_host_cpu_features(True)
        rows, cols = keep["rows"], keep["cols"]
        slab_rows = min(rows, 16 * 96)               # 96 tile rows of 16
        x = keep["x"][:slab_rows].cpu().numpy().reshape(-1)
        o0 = slab_rows // 16
        packed = np.zeros(o0 * cols * 16, np.float32)
        flags = uk.PACK_TYPE_F32F32 | uk.PACK_TRANSPOSE_OUTER
        t0 = time.perf_counter()
        # TRANSPOSE_OUTER: stored [cols][o0][16][1]
        chk.pack(x, 0, cols, 1, packed, 0, o0 * 16, 16, slab_rows, cols, cols, o0, 16, 1,
                 0xBF800000, flags)
        t_pack = time.perf_counter() - t0
        back = np.zeros(slab_rows * cols, np.float32)
        t0 = time.perf_counter()
        chk.unpack(packed, 0, o0 * 16, 16, back, 0, cols, 1, cols, o0, 16, 1, slab_rows, cols,
                   uk.UNPACK_TYPE_F32F32 | uk.UNPACK_TRANSPOSE_OUTER)
        t_un = time.perf_counter() - t0
        ok = bool(np.array_equal(back, x))
        nbytes = 2.0 * slab_rows * cols * 4
        return {"value": round(2 * nbytes / (t_pack + t_un) / 1e9, 3), "unit": "GB/s", "cores": 1,
                "kind": "reference" if have_ref else "port",
                "sample": f"pack + unpack of the first {slab_rows} of {rows} rows, 1 thread "
                          f"({t_pack:.2f} s + {t_un:.2f} s); round trip exact: {ok}"}
    if wl.name.startswith("conv_nchwc"):
        # One image of the batch, single thread, the reference's AVX-512
        # 16x16x16 tile when the host has it (else its generic tile); the GPU
        # result of the same image is compared on the way.
        chk = uk_oracle.Checker("reference" if have_ref else "oracle")
        chk.use_host_cpu_features(True)
        d = {k: keep[k] for k in ("N", "ICo", "OCo", "OH", "OW", "FH", "FW", "k0", "c0")}
        H, W = d["OH"] + d["FH"] - 1, d["OW"] + d["FW"] - 1
        in_s = (d["ICo"] * H * W * d["c0"], H * W * d["c0"], W * d["c0"])
        f_s = (d["ICo"] * d["FH"] * d["FW"] * d["c0"] * d["k0"], d["FH"] * d["FW"] * d["c0"] * d["k0"],
               d["FW"] * d["c0"] * d["k0"])
        o_s = (d["OCo"] * d["OH"] * d["OW"] * d["k0"], d["OH"] * d["OW"] * d["k0"], d["OW"] * d["k0"])
        x = keep["x"][:in_s[0]].cpu().numpy()
        w = keep["w"].cpu().numpy()
        y = np.zeros(o_s[0], np.float32)
        t0 = time.perf_counter()
        chk.conv_nchwc(x, 0, *in_s, w, 0, *f_s, y, 0, *o_s, 1, d["OCo"], d["OH"], d["OW"], d["ICo"],
                       d["FH"], d["FW"], d["k0"], d["c0"], 1, 1, 0x01 | 0x200)
        t = time.perf_counter() - t0
        got = keep["y"][:o_s[0]].cpu().numpy()
        err = float(np.abs(got - y).max() / np.abs(y).max())
        return {"value": round(wl.flops / d["N"] / t / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                "kind": "reference" if have_ref else "port",
                "sample": f"image 0 of {d['N']}, 1 thread ({t:.2f} s), host ISA paths enabled; "
                          f"GPU result of that image: max|gpu-ref|/max|ref| = {err:.2e}"}
    if "lhs4" not in keep or "M1" not in keep and "M" not in keep:
        return None
    dtype = wl.dtype
    if dtype not in ("s8", "f16", "bf16", "f32", "f8", "s16"):
        return None
    kind = "reference" if (have_ref and dtype != "f8") else "port"
    chk = uk_oracle.Checker("reference" if kind == "reference" else "oracle")
    chk.use_host_cpu_features(True)
    M0, N0, K0 = keep["M0"], keep["N0"], keep["K0"]
    if "M1" in keep:
        M1, N1, K1 = keep["M1"], keep["N1"], keep["K1"]
    else:
        M1, N1, K1 = -(-keep["M"] // M0), -(-keep["N"] // N0), keep["K"] // K0
    flags = _mmt4d_type_flag(dtype, uk) | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    lhs = _host_bytes(keep["lhs4"])
    rhs = _host_bytes(keep["rhs4"])
    out = np.zeros(M1 * N1 * M0 * N0, np.int32 if dtype in ("s8", "s16") else np.float32)
    ls, rs, os_ = K1 * M0 * K0, K1 * N0 * K0, N1 * M0 * N0

    def run(m_tiles, n_tiles):
        t0 = time.perf_counter()
        chk.mmt4d_threaded(T, lhs, ls, rhs, rs, out, os_, m_tiles, n_tiles, K1, M0, N0, K0, flags)
        return time.perf_counter() - t0

    # Calibrate on a small rectangle of tiles, then size the sample: whole tile
    # rows when a few of them fit the time budget, else part of T tile rows.
    if M1 >= T:
        n_cal = min(N1, 2 * T)
        t_cal = run(T, n_cal)
        tiles = (T * n_cal / max(t_cal, 1e-4)) * target_seconds
        if tiles >= T * N1:
            rows = int(min(M1, (tiles / N1) // T * T))
            cols = N1
        else:
            rows, cols = T, int(max(n_cal, min(N1, tiles // T)))
        t = run(rows, cols)
        frac, what = rows * cols / (M1 * N1), f"{rows}/{M1} M tile-rows x {cols}/{N1} N tile-columns"
    else:         # one (or few) tile rows: slab of N tile columns
        n_cal = min(N1, 4 * T)
        t_cal = run(M1, n_cal)
        cols = int(max(n_cal, min(N1, n_cal * round(target_seconds / max(t_cal, 1e-4)))))
        t = run(M1, cols)
        frac, what = cols / N1, f"{M1}/{M1} M tile-rows x {cols}/{N1} N tile-columns"
    return {"value": round(wl.ops[[o.name for o in wl.ops].index("mmt4d")].flops * frac / t / 1e12, 6),
            "unit": "TFLOP/s", "cores": T, "kind": kind,
            "sample": f"mmt4d only, on {what} over {T} threads ({t:.2f} s), host ISA paths enabled; "
                      "extrapolated linearly to the whole problem"}


def verify_c2(runner, keep, cpu_out4, slab) -> dict:
    """GPU result of the timed chain against the CPU checker on the slab the
    baseline computed: max|gpu-ref|/max|ref| must be <= 1e-2 (f16 inputs, f32
    accumulation in a different order)."""
    import numpy as np
    M0, N0 = keep["M0"], keep["N0"]
    N1 = -(-keep["N"] // N0)
    n = slab * N1 * M0 * N0
    got = keep["out4"][:n].cpu().numpy()
    want = cpu_out4[:n]
    err = float(np.abs(got - want).max() / np.abs(want).max())
    return {"checked_tile_rows": slab, "max_err_over_max_ref": err, "tolerance": 1e-2,
            "ok": bool(err <= 1e-2)}


def verify_sampled_tiles(wl, n_random: int = 64, seed: int = 0) -> dict:
    """The mmt4d output of a workload, as the timed launches left it in HBM,
    against the CPU oracle on sampled output tiles: the four corners plus
    `n_random` tiles drawn at random, each over all of K (one oracle call with
    M = N = 1 on that tile's panels). s8: bit-exact; floats: max|gpu-ref| /
    max|ref| over the sampled elements against the tolerance of the type."""
    import numpy as np
    from oracle import uk_oracle
    from iree_amd import ukernel as uk

    k = wl.keep
    dtype = wl.dtype
    M0, N0, K0 = k["M0"], k["N0"], k["K0"]
    if "M1" in k:
        M1, N1, K1 = k["M1"], k["N1"], k["K1"]
    else:
        M1, N1, K1 = -(-k["M"] // M0), -(-k["N"] // N0), k["K"] // K0
    es = {"s8": 1, "f8": 1, "f16": 2, "bf16": 2, "f32": 4, "s16": 2}[dtype]
    view = {1: np.uint8, 2: np.uint16, 4: np.uint32}[es]
    chk = uk_oracle.get("oracle")
    lhs = _host_bytes(k["lhs4"]).reshape(M1, K1 * M0 * K0 * es)
    rhs = _host_bytes(k["rhs4"]).reshape(N1, K1 * N0 * K0 * es)
    integer = dtype in ("s8", "s16")
    out_dt = np.int32 if integer else np.float32
    got_all = _host_bytes(k["out4"]).view(out_dt).reshape(M1, N1, M0 * N0)
    rng = np.random.default_rng(seed)
    tiles = {(0, 0), (0, N1 - 1), (M1 - 1, 0), (M1 - 1, N1 - 1)}
    while len(tiles) < min(n_random + 4, M1 * N1):
        tiles.add((int(rng.integers(M1)), int(rng.integers(N1))))
    flags = _mmt4d_type_flag(dtype, uk) | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    exact, max_err, max_ref = True, 0.0, 0.0
    for (m, n) in sorted(tiles):
        want = np.zeros(M0 * N0, out_dt)
        chk.mmt4d(lhs[m].view(view), 0, K1 * M0 * K0, rhs[n].view(view), 0, K1 * N0 * K0, want, 0,
                  M0 * N0, 1, 1, K1, M0, N0, K0, flags)
        got = got_all[m, n]
        if integer:
            exact = exact and bool(np.array_equal(got, want))
        else:
            if not (np.isfinite(got).all() and np.isfinite(want).all()):
                return {"tiles": len(tiles), "ok": False, "error": f"non-finite value in tile ({m}, {n})"}
            max_err = max(max_err, float(np.abs(got - want).max()))
            max_ref = max(max_ref, float(np.abs(want).max()))
    if integer:
        return {"tiles": len(tiles), "bit_exact": exact, "ok": exact}
    tol = {"f16": 1e-2, "bf16": 1e-2, "f8": 2e-2, "f32": 1e-5}[dtype]
    err = max_err / max_ref if max_ref else 0.0
    return {"tiles": len(tiles), "max_err_over_max_ref": float(f"{err:.3e}"), "tolerance": tol,
            "ok": bool(err <= tol)}


# The north-star workloads whose figures are repeated, compactly, in the
# top-level `targets` block at the END of the JSON line.
TARGET_MMT4D = ["s8_mmt4d_8192_k16", "s8_mmt4d_8192_k2", "s8_mmt4d_1024_k2", "bf16_mmt4d_8192_k2",
                "bf16_mmt4d_8192_k8", "f8_mmt4d_8192_k32", "c4_f8_prefill"]
TARGET_PACK = {
    # name: (rows, row_bytes, src_pitch, dst_pitch) of the plain copy that moves
    # the same matrix between the same two pitches
    "c5_pack_f32_12288x12289": (12288, 49152, 49156, 49152),
    "c5_pack_f32_12289x12288": (12288, 49152, 49152, 49216),
    # the prefill's RHS pack (1-byte elements, 16x32 tiles: rows of 8192 bytes both sides)
    "c4_f8_prefill": (28672, 8192, 8192, 8192),
}


def vendor_gemm_context(torch) -> dict:
    """Context, not a baseline: the GEMM that this image's PyTorch dispatches to
    the vendor library (torch.matmul / torch._int_mm / torch._scaled_mm on
    row-major operands, B given as [N][K]) at the sizes of the mmt4d targets, on
    the same device in the same run, as microseconds and as a fraction of the
    same published peaks. It shows where a tuned library sits under this part's
    power limit; its operands are not tiled, so it is not the same interface."""
    out = {}

    def timed(f, n=10):
        for _ in range(3):
            f()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.2:   # clocks settle under load
            f()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            f()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n

    def entry(name, S, peak, f):
        try:
            us = timed(f)
            out[name] = {"us": round(us, 1), "frac": round(2.0 * S ** 3 / us / 1e6 / peak, 4)}
        except Exception as e:   # an op this build of torch does not have
            out[name] = {"error": repr(e)[:120]}

    for dt, nm in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        for S in (4096, 8192):
            x = torch.randn(S, S, device="cuda", dtype=dt)
            y = torch.randn(S, S, device="cuda", dtype=dt)
            entry(f"{nm}_{S}", S, 2500.0, lambda: torch.matmul(x, y.t()))
            del x, y
    S = 8192
    x = torch.randint(-128, 128, (S, S), device="cuda", dtype=torch.int8)
    y = torch.randint(-128, 128, (S, S), device="cuda", dtype=torch.int8)
    entry("s8_8192", S, 5000.0, lambda: torch._int_mm(x, y.t()))
    del x, y
    try:
        x = torch.randn(S, S, device="cuda").to(torch.float8_e4m3fn)
        y = torch.randn(S, S, device="cuda").to(torch.float8_e4m3fn)
        one = torch.tensor(1.0, device="cuda")
        entry("f8_8192", S, 5000.0,
              lambda: torch._scaled_mm(x, y.t(), scale_a=one, scale_b=one, out_dtype=torch.float32))
    except Exception as e:
        out["f8_8192"] = {"error": repr(e)[:120]}
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_f16_chain_4096")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--extra-iters", type=int, default=20)
    ap.add_argument("--sweep", metavar="WORKLOAD", default=None,
                    help="print T(K) of a square mmt4d workload (e.g. s8_mmt4d_8192_k16) under the "
                         "big kernel variants, with a straight-line fit, instead of the JSON line")
    ap.add_argument("--shapes", action="store_true",
                    help="print mmt4d timings over transformer-like M x N x K shapes beside the vendor "
                         "library's GEMM on the same device, instead of the JSON line")
    ap.add_argument("--tiles", action="store_true",
                    help="print, for every mmt4d type on the tile shapes of the reference's CPU kernels, "
                         "the kernel that serves it and its rate at 2048^3, instead of the JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path shards by tile rows with no "
              "exchange step, but no multi-GPU figure is produced); use --gpus 1",
              file=sys.stderr)
        return 2

    import torch
    from iree_amd import runner as rn

    torch.cuda.set_device(0)
    R = rn.Runner(seed=0)
    if args.sweep:
        print("command: python bench.py --sweep " + args.sweep)
        print(R.k_sweep(args.sweep))
        R.close()
        return 0
    if args.tiles:
        print("command: python bench.py --tiles")
        print(R.tile_survey())
        R.close()
        return 0
    if args.shapes:
        print("command: python bench.py --shapes")
        print(R.shape_survey())
        R.close()
        return 0
    wl = R.workload(args.workload)
    dominant = "mmt4d" if any(o.name == "mmt4d" for o in wl.ops) else wl.ops[0].name
    sec_per_step, sec_per_step_events, dom_us = R.run_steps(wl, args.steps, args.warmup, dominant)
    dom = next(o for o in wl.ops if o.name == dominant)
    roof = R.roofline(dom, dom_us)
    roof["kernel"] = dom.kernel
    roof["avg_us"] = round(dom_us, 2)
    roof["traffic"], roof["traffic_source"] = recorded_traffic(args.workload, dominant, dom.kernel)

    per_kernel = {}
    for op in wl.ops:
        avg, mn, med = R.time_op(op, max(5, min(args.steps, 30)))
        r = R.roofline(op, avg)
        per_kernel[op.name] = {"kernel": op.kernel, "avg_us": round(avg, 2), "min_us": round(mn, 2),
                               "median_us": round(med, 2),
                               "achieved": r["achieved"], "unit": r["unit"], "frac": r["frac"]}
        if r["bound"] == "hbm" and op.bytes >= COLD_FROM_BYTES and not op.external \
                and not args.workload.endswith("_cold"):
            # (the same launches with the memory-side cache emptied before each)
            cavg, cmn, cmed = R.time_op(op, max(5, min(args.steps, 30) // 2), cold=True)
            rc = R.roofline(op, cavg)
            per_kernel[op.name].update({"cold_avg_us": round(cavg, 2), "cold_min_us": round(cmn, 2),
                                        "cold_achieved": rc["achieved"], "cold_frac": rc["frac"]})

    if wl.flops:
        metric = ("conv_nchwc TFLOP/s" if dominant == "conv"
                  else "mmt4d TFLOP/s over the pack->mmt4d->unpack chain")
        unit = "TFLOP/s"
        value = wl.flops / sec_per_step / 1e12
    else:
        metric, unit = "pack/unpack HBM GB/s", "GB/s"
        value = wl.bytes / sec_per_step / 1e9

    result = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 4),
        "ms_per_step_with_kernel_events": round(sec_per_step_events * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": wl.dtype,
        "data": "synthetic (seeded, generated in HBM)",
        "config": {"workload": wl.name, "description": wl.description},
        "roofline": roof, "kernels": per_kernel,
        "measured_copy_GBps": round(R.measured_copy_gbps(), 1),
        "host": cpu_info(),
    }
    # Ceilings measured on this device in this run: a loop of nothing but the
    # type's MFMA instruction (random operands; and zeros for s8, which shows
    # what the power limit costs), beside the published peaks.
    peaks = {dt: round(R.measured_mfma_peak(dt), 1) for dt in ("s8", "f8", "f16", "bf16", "f32")}
    peaks["s8_zero_operands"] = round(R.measured_mfma_peak("s8", zeros=True), 1)
    result["measured_mfma_only_TOPS"] = peaks
    # The shader clock those rates imply: rate / (1024 SIMDs x operations per SIMD
    # and clock), the published peak being that product at 2.4 GHz.
    result["measured_mfma_only_clock_GHz"] = {
        dt: round(2.4 * v / rn.PEAK_TFLOPS["s8" if dt.startswith("s8") else dt], 3) for dt, v in peaks.items()}
    # What one wave per SIMD can feed the matrix pipe against what two can (s8
    # loop with its MFMAs as assembly, one workgroup per CU; zeros: free of the
    # power limit).
    wz, wr = R.measured_mfma_waves(zeros=True), R.measured_mfma_waves(zeros=False)
    result["measured_mfma_only_waves_per_simd_TOPS"] = {
        "zero_operands": {"two": round(wz[2], 1), "one": round(wz[1], 1), "one_over_two": round(wz[1] / wz[2], 3)},
        "random_operands": {"two": round(wr[2], 1), "one": round(wr[1], 1), "one_over_two": round(wr[1] / wr[2], 3)}}
    result["vendor_gemm_same_device"] = vendor_gemm_context(torch)
    if roof["bound"] == "mfma" and wl.dtype in peaks and peaks[wl.dtype] > 0:
        # the same kernel against the ceiling measured in this run
        roof["of_measured_mfma_only"] = round(roof["achieved"] / peaks[wl.dtype], 4)

    if not args.no_cpu and args.workload.startswith("c2_f16_chain"):
        base, cpu_out4, slab = cpu_baseline_c2(wl.keep)
        result["cpu_baseline"] = base
        result["parity"] = verify_c2(R, wl.keep, cpu_out4, slab)
    else:
        result["cpu_baseline"] = None

    if not args.no_extra:
        extra = {}
        del wl
        for name in EXTRA_WORKLOADS:
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            w = R.workload(name)
            entry = {"description": w.description, "kernels": {}}
            total_us = 0.0
            for op in w.ops:
                avg, mn, med = R.time_op(op, args.extra_iters)
                r = R.roofline(op, avg)
                total_us += avg
                entry["kernels"][op.name] = {
                    "kernel": op.kernel, "avg_us": round(avg, 2), "min_us": round(mn, 2),
                    "median_us": round(med, 2),
                    "bound": r["bound"], "achieved": r["achieved"], "unit": r["unit"],
                    "frac": r["frac"]}
                if r["bound"] == "hbm" and op.bytes >= COLD_FROM_BYTES and not op.external \
                        and not name.endswith("_cold"):
                    # The launches above run on the same buffers one after the
                    # other and find part of them in the memory-side cache; here
                    # the cache is emptied before every launch.
                    cavg, cmn, cmed = R.time_op(op, max(5, args.extra_iters // 2), cold=True)
                    rc = R.roofline(op, cavg)
                    entry["kernels"][op.name].update({
                        "cold_avg_us": round(cavg, 2), "cold_min_us": round(cmn, 2),
                        "cold_achieved": rc["achieved"], "cold_frac": rc["frac"]})
            if w.flops:
                # sum of the kernels' device times (no launch gaps)
                entry["chain_TFLOPs"] = round(w.flops / (total_us * 1e-6) / 1e12, 3)
            if not args.no_cpu and not name.endswith("_zeros"):
                try:
                    entry["cpu_baseline"] = cpu_baseline_extra(w)
                except Exception as e:  # the baseline is a reported aside, never fatal
                    entry["cpu_baseline"] = {"error": repr(e)}
            if not args.no_cpu and (name in TARGET_MMT4D or name.startswith("s16_mmt4d_")):
                entry["parity"] = verify_sampled_tiles(w)
            if name in TARGET_PACK:
                rows, row_bytes, sp, dp = TARGET_PACK[name]
                gbps = R.copy2d_ceiling_gbps(rows, row_bytes, sp, dp)
                whole = R.last_copy2d_whole_lines_gbps
                cold_gbps = R.copy2d_ceiling_gbps(rows, row_bytes, sp, dp, iters=3, cold=True)
                entry["copy2d_ceiling"] = {
                    "GBps": round(gbps, 1), "frac": round(gbps / rn.PEAK_HBM_GBPS, 4),
                    "cold_frac": round(cold_gbps / rn.PEAK_HBM_GBPS, 4),
                    "whole_lines_only_frac": round(whole / rn.PEAK_HBM_GBPS, 4),
                    "what": f"plain copy of {rows} rows x {row_bytes} B, pitch {sp} -> {dp} B"}
                if "unpack" in w.ops[-1].name:
                    # unpack moves the matrix the other way: its ceiling is
                    # the copy into the 2-D side's pitch
                    back = R.copy2d_ceiling_gbps(rows, row_bytes, dp, sp)
                    back_whole = R.last_copy2d_whole_lines_gbps
                    cold_back = R.copy2d_ceiling_gbps(rows, row_bytes, dp, sp, iters=3, cold=True)
                    entry["copy2d_ceiling_unpack"] = {
                        "GBps": round(back, 1), "frac": round(back / rn.PEAK_HBM_GBPS, 4),
                        "cold_frac": round(cold_back / rn.PEAK_HBM_GBPS, 4),
                        "whole_lines_only_frac": round(back_whole / rn.PEAK_HBM_GBPS, 4),
                        "what": f"plain copy of {rows} rows x {row_bytes} B, pitch {dp} -> {sp} B"}
                keep = w.keep
                if "back" in keep:
                    entry["parity"] = {"round_trip_bit_exact": bool(
                        torch.equal(keep["back"].view(keep["rows"], keep["cols"]), keep["x"]))}
            if name == "pack_operand_forms":
                # every packed operand against the same regrouping written with
                # torch's reshape and permute, bit for bit
                ok = {}
                for oname, x, out, X0, K0, kn in w.keep["forms"]:
                    rows, cols = x.shape
                    if kn:
                        want = x.view(rows // K0, K0, cols // X0, X0).permute(2, 0, 3, 1)
                    else:
                        want = x.view(rows // X0, X0, cols // K0, K0).permute(0, 2, 1, 3)
                    ok[oname] = bool(torch.equal(out.view(want.shape), want.contiguous()))
                entry["parity"] = {"equals_reshape_permute": ok, "ok": all(ok.values())}
            extra[name] = entry
            del w
        result["extra"] = extra

        # ---- targets: compact, last in the line -------------------------------
        targets = {"_": "frac: of the published peak (s8/f8 5000, f16/bf16 2500 TOP/s, HBM 8000 GB/s); "
                        "of_mfma_only / of_copy2d: of the ceiling measured in this run"}
        for name in TARGET_MMT4D:
            e = extra.get(name)
            if not e:
                continue
            kk = e["kernels"]["mmt4d"]
            dt = name.split("_")[0] if not name.startswith("c4") else "f8"
            traffic, traffic_source = recorded_traffic(name, "mmt4d", kk["kernel"])
            t = {"kernel": kk["kernel"].replace("mmt4d_mfma_", ""), "us": kk["avg_us"],
                 "TOPS": round(kk["achieved"], 1), "frac": round(kk["frac"], 3),
                 "of_mfma_only": round(kk["achieved"] / peaks[dt], 3),
                 # the same object as the headline's `roofline`, for this workload's mmt4d kernel
                 "roofline": {"bound": kk["bound"], "achieved": kk["achieved"],
                              "peak": rn.PEAK_TFLOPS[dt], "unit": kk["unit"], "frac": kk["frac"],
                              "traffic": traffic, "traffic_source": traffic_source,
                              "of_measured_mfma_only": round(kk["achieved"] / peaks[dt], 4)}}
            if "parity" in e:
                par = e["parity"]
                t["parity"] = ("bit-exact on %d sampled tiles" % par["tiles"] if par.get("bit_exact")
                               else ("MISMATCH" if "bit_exact" in par else
                                     par.get("error") or
                                     "err %.1e <= %g: %s" % (par["max_err_over_max_ref"], par["tolerance"], par["ok"])))
            cb = e.get("cpu_baseline") or {}
            if "value" in cb:
                t["cpu"] = "%.3g %s, %d thr, %s" % (cb["value"], cb["unit"], cb["cores"], cb["kind"])
            for pk in ("pack_lhs", "pack_rhs"):
                if pk in e["kernels"]:
                    t[pk + "_frac"] = round(e["kernels"][pk]["frac"], 3)
            if "copy2d_ceiling" in e:
                t["copy2d_frac"] = round(e["copy2d_ceiling"]["frac"], 3)
            targets[name] = t
        # The decode layer (HBM-bound: its weights stream once per launch). `warm`:
        # the benchmark's repeated launches find the 58.7 MB of weights in the 256 MB
        # memory-side cache; `cold`: launches rotate over eight copies of the weights,
        # so every launch streams them from HBM - the figure a serving loop sees.
        for name, label in (("c3_s8_decode", "warm"), ("c3_s8_decode_cold", "cold"),
                            ("c3_s8_decode_fused", "warm"), ("c3_s8_decode_fused_cold", "cold"),
                            ("c3_s8_decode_down", "warm")):
            e = extra.get(name)
            if not e:
                continue
            kk = e["kernels"]["mmt4d"]
            traffic, traffic_source = recorded_traffic(name, "mmt4d", kk["kernel"])
            targets[name] = {"kernel": kk["kernel"].replace("mmt4d_mfma_", ""), "weights": label,
                             "us": kk["avg_us"], "GBps": round(kk["achieved"], 1),
                             "frac": round(kk["frac"], 3),
                             "roofline": {"bound": "hbm", "achieved": kk["achieved"],
                                          "peak": rn.PEAK_HBM_GBPS, "unit": "GB/s", "frac": kk["frac"],
                                          "traffic": traffic, "traffic_source": traffic_source}}
        e = extra.get("s16_mmt4d_4096_k2")
        if e:
            kk = e["kernels"]["mmt4d"]
            targets["s16_mmt4d_4096_k2"] = {
                "kernel": kk["kernel"], "us": kk["avg_us"], "TOPS": round(kk["achieved"], 1),
                "frac": round(kk["frac"], 3),
                "roofline": {"bound": "mfma", "achieved": kk["achieved"], "peak": rn.PEAK_TFLOPS["s16"],
                             "unit": kk["unit"], "frac": kk["frac"], "traffic": None,
                             "what": "no 16-bit integer matrix instruction: a 16 x 16-bit product runs as four "
                                     "8 x 8-bit products, so the peak is a quarter of the int8 one"}}
        for name in TARGET_PACK:
            e = extra.get(name)
            if not e or "pack" not in e["kernels"]:
                continue
            targets[name] = {"pack_frac": round(e["kernels"]["pack"]["frac"], 3),
                             "unpack_frac": round(e["kernels"]["unpack"]["frac"], 3),
                             "copy2d_frac": round(e["copy2d_ceiling"]["frac"], 3),
                             "copy2d_unpack_frac": round(e["copy2d_ceiling_unpack"]["frac"], 3),
                             # the same four with the memory-side cache emptied between launches
                             "cold": {"pack_frac": e["kernels"]["pack"].get("cold_frac"),
                                      "unpack_frac": e["kernels"]["unpack"].get("cold_frac"),
                                      "copy2d_frac": e["copy2d_ceiling"]["cold_frac"],
                                      "copy2d_unpack_frac": e["copy2d_ceiling_unpack"]["cold_frac"]},
                             "round_trip_bit_exact": e["parity"]["round_trip_bit_exact"]}
        e = extra.get("pack_operand_forms")
        if e:
            ks = e["kernels"].values()
            targets["pack_operand_forms"] = {
                "kernels": sorted({k["kernel"] for k in ks}),
                # launches on the same buffers (source in the memory-side cache) / that cache emptied before each
                "frac_same_buffers": [round(min(k["frac"] for k in ks), 3), round(max(k["frac"] for k in ks), 3)],
                "frac_cold": [round(min(k.get("cold_frac", float("nan")) for k in ks), 3),
                              round(max(k.get("cold_frac", float("nan")) for k in ks), 3)],
                "equals_reshape_permute": e["parity"]["ok"]}
        result["targets"] = targets

    R.close()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
