"""One-GPU runner for the pack / mmt4d / unpack ukernels: builds the benchmark
workloads from seeded synthetic tensors resident in HBM, times each kernel with
HIP events on the stream the kernels are launched on, and reports TOPS /
TFLOP/s and GB/s next to the MI355X roofline.

Conventions follow the reference's own benchmarks with one stated difference:
  * mmt4d work = 2*M*N*K on the logical (unpadded) sizes
    (runtime/src/iree/builtins/ukernel/tools/mmt4d_benchmark.c:82-84);
  * pack/unpack bytes = bytes that must be read + bytes that must be written
    (the reference counts the output buffer only,
    tools/pack_benchmark.c:97-101; read+write is what bounds an HBM kernel).

PyTorch is used for device memory, streams and events only.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Callable

from . import ukernel as uk

# Published MI355X peaks (dense).
PEAK_HBM_GBPS = 8000.0
PEAK_TFLOPS = {"s8": 5000.0, "f8": 5000.0, "f16": 2500.0, "bf16": 2500.0, "f32": 157.3,
               # s16 has no matrix instruction of its own: a 16 x 16-bit product is four
               # 8 x 8-bit products on the int8 matrix instruction, so a quarter of its peak.
               "s16": 1250.0}


@dataclasses.dataclass
class Op:
    name: str                 # e.g. "mmt4d", "pack_lhs"
    launch: Callable[[], None]
    flops: float = 0.0        # algorithmic ops per launch
    bytes: float = 0.0        # algorithmic HBM bytes per launch (read + write)
    bound: str = "hbm"        # "hbm" | "mfma"
    dtype: str = ""
    kernel: str = ""          # filled after the first launch
    external: bool = False    # True: not a ukernel call (a harness-side torch op)


@dataclasses.dataclass
class Workload:
    name: str
    description: str
    ops: list
    flops: float              # logical 2*M*N*K of the whole step (0 for pure movement)
    bytes: float              # algorithmic bytes of the whole step
    dtype: str
    keep: dict                # tensors and sizes for verification


def _torch():
    import torch
    return torch


class Runner:
    def __init__(self, seed: int = 0):
        torch = _torch()
        if not torch.cuda.is_available():
            raise RuntimeError("the runner needs a GPU")
        self.torch = torch
        self.lib = uk.load()
        self.stream = torch.cuda.Stream()
        self.seed = seed
        self.lib.set_stream(self.stream.cuda_stream)
        self.lib.set_pointer_mode(uk.POINTER_MODE_DEVICE)
        self.settle_seconds = 0.05

    def close(self):
        self.lib.set_stream(None)
        self.lib.set_pointer_mode(uk.POINTER_MODE_AUTO)

    # ------------------------------------------------------------ generators
    def _gen(self, tensor_id: int):
        g = self.torch.Generator(device="cuda")
        g.manual_seed((self.seed << 8) ^ tensor_id)
        return g

    def normal(self, shape, dtype, tensor_id, scale=1.0):
        t = self.torch.randn(shape, generator=self._gen(tensor_id), device="cuda",
                             dtype=self.torch.float32)
        if scale != 1.0:
            t *= scale
        return t.to(dtype)

    def normal_f8(self, shape, tensor_id):
        """N(0,1) scaled so that the sample maximum maps to 448, cast to
        E4M3FN with round-to-nearest-even; stored as bytes."""
        torch = self.torch
        t = torch.randn(shape, generator=self._gen(tensor_id), device="cuda",
                        dtype=torch.float32)
        t *= 448.0 / t.abs().max()
        return t.to(torch.float8_e4m3fn).view(torch.uint8)

    def uniform_s8(self, shape, tensor_id):
        return self.torch.randint(-128, 128, shape, generator=self._gen(tensor_id),
                                  device="cuda", dtype=self.torch.int8)

    def clipped_normal_s8(self, shape, tensor_id, sigma):
        t = self.torch.randn(shape, generator=self._gen(tensor_id), device="cuda",
                             dtype=self.torch.float32) * sigma
        return t.round().clamp(-128, 127).to(self.torch.int8)

    def empty(self, n, dtype):
        return self.torch.empty(n, device="cuda", dtype=dtype)

    # -------------------------------------------------------------- op makers
    def _pack_op(self, name, src, rows, cols, dst, tile0, tile1, type_flag, es,
                 pad=0, transpose_outer=False):
        o0, o1 = -(-rows // tile0), -(-cols // tile1)
        flags = type_flag | (uk.PACK_TRANSPOSE_OUTER if transpose_outer else 0)
        s0, s1 = (o1, o0) if transpose_outer else (o0, o1)
        lib = self.lib
        sp, dp = src.data_ptr(), dst.data_ptr()

        def launch():
            lib.pack(sp, 0, cols, 1, dp, 0, s1 * tile0 * tile1, tile0 * tile1, rows,
                     cols, s0, s1, tile0, tile1, pad, flags)
        return Op(name, launch, 0.0, float(rows * cols * es + o0 * o1 * tile0 * tile1 * es),
                  "hbm")

    def _unpack_op(self, name, src, dst, rows, cols, tile0, tile1, type_flag, es,
                   transpose_outer=False):
        o0, o1 = -(-rows // tile0), -(-cols // tile1)
        flags = type_flag | (uk.UNPACK_TRANSPOSE_OUTER if transpose_outer else 0)
        s0, s1 = (o1, o0) if transpose_outer else (o0, o1)
        lib = self.lib
        sp, dp = src.data_ptr(), dst.data_ptr()

        def launch():
            lib.unpack(sp, 0, s1 * tile0 * tile1, tile0 * tile1, dp, 0, cols, 1, s0,
                       s1, tile0, tile1, rows, cols, flags)
        # Only the bytes of tiles' valid elements have to move.
        return Op(name, launch, 0.0, float(2 * rows * cols * es), "hbm")

    def _mmt4d_op(self, lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0, type_flag, dtype,
                  in_es, accumulate=False, logical=None):
        flags = type_flag | (uk.MMT4D_ACCUMULATE if accumulate else 0)
        lib = self.lib
        lp, rp, op_ = lhs4.data_ptr(), rhs4.data_ptr(), out4.data_ptr()

        def launch():
            lib.mmt4d(lp, 0, K1 * M0 * K0, rp, 0, K1 * N0 * K0, op_, 0, N1 * M0 * N0,
                      M1, N1, K1, M0, N0, K0, flags)
        M, N, K = logical if logical else (M1 * M0, N1 * N0, K1 * K0)
        out_bytes = M1 * N1 * M0 * N0 * 4 * (2 if accumulate else 1)
        nbytes = (M1 * K1 * M0 * K0 + N1 * K1 * N0 * K0) * in_es + out_bytes
        return Op("mmt4d", launch, 2.0 * M * N * K, float(nbytes), "mfma", dtype)

    def _mmt4d_unpack_op(self, lhs4, rhs4, out, M, N, M1, N1, K1, M0, N0, K0, type_flag, dtype,
                         in_es):
        """The fused call: operands tiled, result row-major M x N."""
        lib = self.lib
        lp, rp, op_ = lhs4.data_ptr(), rhs4.data_ptr(), out.data_ptr()

        def launch():
            lib.mmt4d_unpack(lp, 0, K1 * M0 * K0, rp, 0, K1 * N0 * K0, op_, 0, N, M, N,
                             M1, N1, K1, M0, N0, K0, type_flag)
        nbytes = (M1 * K1 * M0 * K0 + N1 * K1 * N0 * K0) * in_es + M * N * 4
        return Op("mmt4d", launch, 2.0 * M * N * K1 * K0, float(nbytes), "mfma", dtype)

    # --------------------------------------------------------------- workloads
    def workload(self, name: str) -> Workload:
        """Builds the named workload. Its tensors are generated by torch on
        torch's current stream while the ops launch on the runner's own: the
        device is synchronized before the workload is handed out, so a first
        launch never reads an operand that is still being generated."""
        wl = self._build_workload(name)
        self.torch.cuda.synchronize()
        return wl

    def _build_workload(self, name: str) -> Workload:
        torch = self.torch
        if name in ("c2_f16_chain_4096", "c2_f16_chain_ragged"):
            M, N, K = (4096, 4096, 4096) if name.endswith("4096") else (4095, 4097, 4096)
            M0 = N0 = K0 = 16
            M1, N1, K1 = -(-M // M0), -(-N // N0), K // K0
            a = self.normal((M, K), torch.float16, 1)
            bt = self.normal((N, K), torch.float16, 2)   # RHS given transposed: [N, K]
            lhs4 = self.empty(M1 * K1 * M0 * K0, torch.float16)
            rhs4 = self.empty(N1 * K1 * N0 * K0, torch.float16)
            out4 = self.empty(M1 * N1 * M0 * N0, torch.float32)
            out = self.empty(M * N, torch.float32)
            ops = [self._pack_op("pack_lhs", a, M, K, lhs4, M0, K0, uk.PACK_TYPE_F16F16, 2),
                   self._pack_op("pack_rhs", bt, N, K, rhs4, N0, K0, uk.PACK_TYPE_F16F16, 2),
                   self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                  uk.MMT4D_TYPE_F16F16F32, "f16", 2, logical=(M, N, K)),
                   self._unpack_op("unpack", out4, out, M, N, M0, N0, uk.UNPACK_TYPE_F32F32, 4)]
            return Workload(name, f"pack->mmt4d->unpack f16xf16->f32 M={M} N={N} K={K} tiles 16x16x16",
                            ops, 2.0 * M * N * K, sum(o.bytes for o in ops), "f16",
                            dict(a=a, bt=bt, lhs4=lhs4, rhs4=rhs4, out4=out4, out=out,
                                 M=M, N=N, K=K, M0=M0, N0=N0, K0=K0))
        if name in ("c2_f16_fused_4096", "c2_f16_fused_ragged"):
            # The same chain with the fused mmt4d + unpack entry point.
            M, N, K = (4096, 4096, 4096) if name.endswith("4096") else (4095, 4097, 4096)
            M0 = N0 = K0 = 16
            M1, N1, K1 = -(-M // M0), -(-N // N0), K // K0
            a = self.normal((M, K), torch.float16, 1)
            bt = self.normal((N, K), torch.float16, 2)
            lhs4 = self.empty(M1 * K1 * M0 * K0, torch.float16)
            rhs4 = self.empty(N1 * K1 * N0 * K0, torch.float16)
            out = self.empty(M * N, torch.float32)
            ops = [self._pack_op("pack_lhs", a, M, K, lhs4, M0, K0, uk.PACK_TYPE_F16F16, 2),
                   self._pack_op("pack_rhs", bt, N, K, rhs4, N0, K0, uk.PACK_TYPE_F16F16, 2),
                   self._mmt4d_unpack_op(lhs4, rhs4, out, M, N, M1, N1, K1, M0, N0, K0,
                                         uk.MMT4D_TYPE_F16F16F32, "f16", 2)]
            return Workload(name, f"pack->fused mmt4d+unpack f16xf16->f32 M={M} N={N} K={K} "
                            "tiles 16x16x16", ops, 2.0 * M * N * K, sum(o.bytes for o in ops),
                            "f16", dict(a=a, bt=bt, lhs4=lhs4, rhs4=rhs4, out=out, M=M, N=N, K=K,
                                        M0=M0, N0=N0, K0=K0))
        if name.startswith("s8_mmt4d_"):
            # s8_mmt4d_<size>_k<K0>[_zeros], tiles 16x16xK0, packed operands
            # filled directly. `_zeros` is a power probe: the same launch on
            # all-zero operands, i.e. the same instructions and memory traffic
            # with next to no switching in the multipliers. What it gains over
            # the uniform-random case is clock the part gives up under load,
            # not kernel structure.
            parts = name.split("_")
            zeros = len(parts) == 5 and parts[4] == "zeros"
            if len(parts) != 4 and not zeros:
                raise ValueError(f"unknown workload {name!r}")
            size, k0 = parts[2], parts[3]
            S, K0 = int(size), int(k0[1:])
            M0 = N0 = 16
            M1 = N1 = S // 16
            K1 = S // K0
            lhs4 = self.uniform_s8((M1 * K1 * M0 * K0,), 3)
            rhs4 = self.uniform_s8((N1 * K1 * N0 * K0,), 4)
            if zeros:
                lhs4.zero_()
                rhs4.zero_()
            out4 = self.empty(M1 * N1 * M0 * N0, torch.int32)
            op = self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                uk.MMT4D_TYPE_S8S8S32, "s8", 1)
            return Workload(name, f"mmt4d s8xs8->s32 {S}^3 tiles 16x16x{K0}" +
                            (" on all-zero operands (power probe)" if zeros else ""), [op], op.flops,
                            op.bytes, "s8", dict(lhs4=lhs4, rhs4=rhs4, out4=out4, M1=M1,
                                                 N1=N1, K1=K1, M0=M0, N0=N0, K0=K0))
        if name.startswith("s16_mmt4d_"):
            # s16 x s16 -> s32 (no 16-bit integer matrix instruction: four 8-bit
            # products per element pair), e.g. the reference's AVX-512 VNNI tile 16x16x2
            _, _, size, k0 = name.split("_")
            S, K0 = int(size), int(k0[1:])
            M0 = N0 = 16
            M1 = N1 = S // 16
            K1 = S // K0
            lhs4 = torch.randint(-32768, 32768, (M1 * K1 * M0 * K0,), generator=self._gen(21),
                                 device="cuda", dtype=torch.int16)
            rhs4 = torch.randint(-32768, 32768, (N1 * K1 * N0 * K0,), generator=self._gen(22),
                                 device="cuda", dtype=torch.int16)
            out4 = self.empty(M1 * N1 * M0 * N0, torch.int32)
            op = self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                uk.MMT4D_TYPE_S16S16S32 | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION,
                                "s16", 2)
            return Workload(name, f"mmt4d s16xs16->s32 {S}^3 tiles 16x16x{K0} (four s8 products per element pair)", [op],
                            op.flops, op.bytes, "s16",
                            dict(lhs4=lhs4, rhs4=rhs4, out4=out4, M1=M1, N1=N1, K1=K1,
                                 M0=M0, N0=N0, K0=K0))
        if name.startswith("bf16_mmt4d_"):
            _, _, size, k0 = name.split("_")
            S, K0 = int(size), int(k0[1:])
            M0 = N0 = 16
            M1 = N1 = S // 16
            K1 = S // K0
            lhs4 = self.normal((M1 * K1 * M0 * K0,), torch.bfloat16, 5)
            rhs4 = self.normal((N1 * K1 * N0 * K0,), torch.bfloat16, 6)
            out4 = self.empty(M1 * N1 * M0 * N0, torch.float32)
            op = self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                uk.MMT4D_TYPE_BF16BF16F32, "bf16", 2)
            return Workload(name, f"mmt4d bf16xbf16->f32 {S}^3 tiles 16x16x{K0}", [op],
                            op.flops, op.bytes, "bf16",
                            dict(lhs4=lhs4, rhs4=rhs4, out4=out4, M1=M1, N1=N1, K1=K1,
                                 M0=M0, N0=N0, K0=K0))
        if name.startswith("f8_mmt4d_"):
            _, _, size, k0 = name.split("_")
            S, K0 = int(size), int(k0[1:])
            M0 = N0 = 16
            M1 = N1 = S // 16
            K1 = S // K0
            lhs4 = self.normal_f8((M1 * K1 * M0 * K0,), 17)
            rhs4 = self.normal_f8((N1 * K1 * N0 * K0,), 18)
            out4 = self.empty(M1 * N1 * M0 * N0, torch.float32)
            op = self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, "f8", 1)
            return Workload(name, f"mmt4d f8E4M3FN->f32 {S}^3 tiles 16x16x{K0}", [op],
                            op.flops, op.bytes, "f8",
                            dict(lhs4=lhs4, rhs4=rhs4, out4=out4, M1=M1, N1=N1, K1=K1,
                                 M0=M0, N0=N0, K0=K0))
        if name.startswith("f32_mmt4d_"):
            _, _, size, k0 = name.split("_")
            S, K0 = int(size), int(k0[1:])
            M0 = N0 = 16
            M1 = N1 = S // 16
            K1 = S // K0
            lhs4 = self.normal((M1 * K1 * M0 * K0,), torch.float32, 13)
            rhs4 = self.normal((N1 * K1 * N0 * K0,), torch.float32, 14)
            out4 = self.empty(M1 * N1 * M0 * N0, torch.float32)
            op = self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                uk.MMT4D_TYPE_F32F32F32, "f32", 4)
            return Workload(name, f"mmt4d f32xf32->f32 {S}^3 tiles 16x16x{K0}", [op],
                            op.flops, op.bytes, "f32",
                            dict(lhs4=lhs4, rhs4=rhs4, out4=out4, M1=M1, N1=N1, K1=K1,
                                 M0=M0, N0=N0, K0=K0))
        if name in ("c3_s8_decode", "c3_s8_decode_down"):
            # Decode-shaped quantized linear layer: 16 activations rows padded to
            # M0=32, weights [14336, 4096] pre-packed once (not timed), ACCUMULATE
            # into a seeded s32 buffer. `_down` is its mate in a transformer MLP,
            # the projection back (weights [4096, 14336]): few output blocks and a
            # long K, the shape the K split over workgroups is for.
            Mlog, K, N = (16, 4096, 14336) if name == "c3_s8_decode" else (16, 14336, 4096)
            M0, N0, K0 = 32, 16, 8
            M1, N1, K1 = 1, N // N0, K // K0
            act = self.clipped_normal_s8((Mlog, K), 7, 40.0)
            w = self.uniform_s8((N, K), 8)
            lhs4 = self.empty(M1 * K1 * M0 * K0, torch.int8)
            rhs4 = self.empty(N1 * K1 * N0 * K0, torch.int8)
            out4 = torch.randint(-2 ** 15, 2 ** 15, (M1 * N1 * M0 * N0,),
                                 generator=self._gen(9), device="cuda", dtype=torch.int32)
            pack_w = self._pack_op("pack_weights", w, N, K, rhs4, N0, K0, uk.PACK_TYPE_I8I8, 1)
            pack_w.launch()   # once, outside any timing
            pack_a = self._pack_op("pack_act", act, Mlog, K, lhs4, M0, K0, uk.PACK_TYPE_I8I8, 1)
            pack_a.launch()
            op = self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                uk.MMT4D_TYPE_S8S8S32, "s8", 1, accumulate=True,
                                logical=(Mlog, N, K))
            op.bound = "hbm"
            # The layer's epilogue is not a ukernel: per-row (activation) and
            # per-column (weight) scales applied to the s32 accumulators of the
            # 16 real rows, out[m][n] = float(acc[m][n]) * scale_m[m] * scale_n[n],
            # as one torch expression on the tiled buffer.
            scale_m = torch.rand(Mlog, generator=self._gen(15), device="cuda") * 0.02 + 0.001
            scale_n = torch.rand(N, generator=self._gen(16), device="cuda") * 0.02 + 0.001
            y = torch.empty(Mlog, N, device="cuda", dtype=torch.float32)
            acc_view = out4.view(N1, M0, N0)[:, :Mlog, :].permute(1, 0, 2)  # [m][n1][n0]
            scale = (scale_m[:, None] * scale_n[None, :]).view(Mlog, N1, N0)
            y_view = y.view(Mlog, N1, N0)
            stream = self.stream

            def epilogue():
                with torch.cuda.stream(stream):
                    torch.mul(acc_view, scale, out=y_view)  # one kernel: s32 * f32 -> f32
            ep = Op("scale_epilogue", epilogue, 0.0, float(Mlog * N * 8), "hbm", "f32",
                    kernel="torch (harness, not a ukernel)", external=True)
            return Workload(name, f"mmt4d s8 decode M=16(32) K={K} N={N} tiles 32x16x8 ACCUMULATE "
                            "+ per-row/per-column scale epilogue",
                            [op, ep], op.flops, op.bytes, "s8",
                            dict(act=act, w=w, lhs4=lhs4, rhs4=rhs4, out4=out4, y=y, scale_m=scale_m,
                                 scale_n=scale_n, M1=M1, N1=N1, K1=K1, M0=M0, N0=N0, K0=K0))
        if name == "c3_s8_decode_fused":
            # The same layer through the fused entry point: accumulators read
            # from the tiled s32 buffer, result scaled into the row-major f32
            # matrix by the mmt4d kernel itself (no separate epilogue pass).
            base = self._build_workload("c3_s8_decode")
            t = base.keep
            Mlog, N = t["act"].shape[0], t["w"].shape[0]
            M1, N1, K1, M0, N0, K0 = (t[k] for k in ("M1", "N1", "K1", "M0", "N0", "K0"))
            y = torch.empty(Mlog, N, device="cuda", dtype=torch.float32)
            lib = self.lib
            ptrs = [t[k].data_ptr() for k in ("lhs4", "rhs4", "out4", "scale_m", "scale_n")]
            yp = y.data_ptr()
            flags = uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE

            def launch():
                lib.mmt4d_dequant_unpack(ptrs[0], 0, K1 * M0 * K0, ptrs[1], 0, K1 * N0 * K0,
                                         ptrs[2], 0, N1 * M0 * N0, yp, 0, N, Mlog, N,
                                         ptrs[3], ptrs[4], M1, N1, K1, M0, N0, K0, flags)
            nbytes = (M1 * K1 * M0 * K0 + N1 * K1 * N0 * K0 + M1 * N1 * M0 * N0 * 4 +
                      Mlog * N * 4 + (Mlog + N) * 4)
            op = Op("mmt4d", launch, base.flops, float(nbytes), "hbm", "s8")
            tensors = dict(t)
            tensors["y_fused"] = y
            return Workload(name, "fused mmt4d + dequantizing unpack, s8 decode M=16(32) K=4096 N=14336 "
                            "tiles 32x16x8 ACCUMULATE, per-row/per-column scales",
                            [op], base.flops, float(nbytes), "s8", tensors)
        if name in ("c3_s8_decode_cold", "c3_s8_decode_fused_cold"):
            # The decode layer with its weights streamed from HBM on every
            # launch: the 58.7 MB of packed weights of one layer stay in the
            # 256 MB memory-side cache between a benchmark's repeated launches,
            # which a serving loop that walks through its layers never sees.
            # Here consecutive launches rotate over COLD_COPIES distinct copies
            # of the packed weights (more than the cache holds in total), so
            # each launch reads weights that have long been evicted.
            COLD_COPIES = 8
            fused = name == "c3_s8_decode_fused_cold"
            base = self._build_workload("c3_s8_decode_fused" if fused else "c3_s8_decode")
            t = base.keep
            M1, N1, K1, M0, N0, K0 = (t[k] for k in ("M1", "N1", "K1", "M0", "N0", "K0"))
            copies = [t["rhs4"]] + [t["rhs4"].clone() for _ in range(COLD_COPIES - 1)]
            rps = [c.data_ptr() for c in copies]
            state = {"i": 0}
            lib = self.lib
            lp, accp = t["lhs4"].data_ptr(), t["out4"].data_ptr()
            flags = uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE
            if fused:
                Mlog, N = t["act"].shape[0], t["w"].shape[0]
                yp, smp, snp = t["y_fused"].data_ptr(), t["scale_m"].data_ptr(), t["scale_n"].data_ptr()

                def launch():
                    state["i"] = (state["i"] + 1) % COLD_COPIES
                    lib.set_streamed_weights(True)   # what a serving loop says once per thread
                    lib.mmt4d_dequant_unpack(lp, 0, K1 * M0 * K0, rps[state["i"]], 0, K1 * N0 * K0,
                                             accp, 0, N1 * M0 * N0, yp, 0, N, Mlog, N,
                                             smp, snp, M1, N1, K1, M0, N0, K0, flags)
                    lib.set_streamed_weights(False)
            else:
                def launch():
                    state["i"] = (state["i"] + 1) % COLD_COPIES
                    lib.set_streamed_weights(True)
                    lib.mmt4d(lp, 0, K1 * M0 * K0, rps[state["i"]], 0, K1 * N0 * K0, accp, 0,
                              N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags)
                    lib.set_streamed_weights(False)
            src = base.ops[0]
            op = Op("mmt4d", launch, src.flops, src.bytes, "hbm", "s8")
            tensors = dict(t)
            tensors["weight_copies"] = copies
            return Workload(name, base.description + f"; weights rotate over {COLD_COPIES} copies "
                            f"({COLD_COPIES * copies[0].numel() / 1e6:.0f} MB): every launch streams them from HBM, "
                            "and says so (iree_uk_amd_set_streamed_weights)",
                            [op], base.flops, src.bytes, "s8", tensors)
        if name == "c4_f8_prefill":
            M, K, N = 2048, 8192, 28672
            M0, N0, K0 = 16, 16, 32
            M1, N1, K1 = M // M0, N // N0, K // K0
            a = self.normal_f8((M, K), 10)
            bt = self.normal_f8((N, K), 11)
            lhs4 = self.empty(M * K, torch.uint8)
            rhs4 = self.empty(N * K, torch.uint8)
            out4 = self.empty(M * N, torch.float32)
            ops = [self._pack_op("pack_lhs", a, M, K, lhs4, M0, K0, uk.PACK_TYPE_I8I8, 1),
                   self._pack_op("pack_rhs", bt, N, K, rhs4, N0, K0, uk.PACK_TYPE_I8I8, 1),
                   self._mmt4d_op(lhs4, rhs4, out4, M1, N1, K1, M0, N0, K0,
                                  uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, "f8", 1)]
            return Workload(name, "pack+pack+mmt4d f8E4M3FN->f32 M=2048 K=8192 N=28672 tiles 16x16x32",
                            ops, 2.0 * M * N * K, sum(o.bytes for o in ops), "f8",
                            dict(a=a, bt=bt, lhs4=lhs4, rhs4=rhs4, out4=out4, M=M, N=N, K=K,
                                 M1=M1, N1=N1, K1=K1, M0=M0, N0=N0, K0=K0))
        if name == "conv_nchwc_f32_n16_56x56_c256_k256_3x3":
            # iree_uk_conv_nchwc at the reference's tuned tile shape (k0 = c0 = 16):
            # a 3x3 stride-1 layer, 256 -> 256 channels, 56x56 outputs, batch 16.
            N, ICo, OCo, OH, OW, FH, FW, k0, c0 = 16, 16, 16, 56, 56, 3, 3, 16, 16
            H, W = OH + FH - 1, OW + FW - 1
            x = self.normal((N * ICo * H * W * c0,), torch.float32, 20)
            w = self.normal((OCo * ICo * FH * FW * c0 * k0,), torch.float32, 21)
            y = self.empty(N * OCo * OH * OW * k0, torch.float32)
            lib = self.lib
            xp, wp, yp = x.data_ptr(), w.data_ptr(), y.data_ptr()
            in_strides = (ICo * H * W * c0, H * W * c0, W * c0)
            f_strides = (ICo * FH * FW * c0 * k0, FH * FW * c0 * k0, FW * c0 * k0)
            out_strides = (OCo * OH * OW * k0, OH * OW * k0, OW * k0)

            def launch():
                lib.conv_nchwc(xp, 0, *in_strides, wp, 0, *f_strides, yp, 0, *out_strides,
                               N, OCo, OH, OW, ICo, FH, FW, k0, c0, 1, 1, 0x01)
            flops = 2.0 * N * OCo * k0 * OH * OW * ICo * c0 * FH * FW
            nbytes = 4.0 * (x.numel() + w.numel() + y.numel())
            op = Op("conv", launch, flops, nbytes, "mfma", "f32")
            return Workload(name, "conv_nchwc f32 N=16 256->256 channels 56x56 outputs 3x3 stride 1, "
                            "tiles k0=16 c0=16", [op], flops, nbytes, "f32",
                            dict(x=x, w=w, y=y, N=N, ICo=ICo, OCo=OCo, OH=OH, OW=OW, FH=FH, FW=FW,
                                 k0=k0, c0=c0))
        if name == "pack_operand_forms":
            # Matmul operands on their way into tiles, in the forms that need an
            # element-wise transposition: the row-major [K][N] right-hand side
            # (TRANSPOSE_INNER + TRANSPOSE_OUTER -> [N1][K1][N0][K0],
            # tests/e2e/linalg/pack_i8.mlir:48-68) for the tile shapes of the
            # other workloads, and the reference's 16x2 s8 tile from [M][K].
            # Every form moves more than the 256 MB memory-side cache holds, but
            # its source alone fits, and launches on the same buffers one after
            # the other read it from there: bench.py times each form a second
            # time with that cache emptied before every launch.
            forms = [  # (op name, torch dtype, pack type, element bytes, rows, cols, N0 or M0, K0, [K][N]?)
                ("rhs_kn_f16_16x16", torch.float16, uk.PACK_TYPE_F16F16, 2, 8192, 16384, 16, 16, True),
                ("rhs_kn_s8_16x8", torch.int8, uk.PACK_TYPE_I8I8, 1, 8192, 28672, 16, 8, True),
                ("rhs_kn_f8_16x32", torch.int8, uk.PACK_TYPE_I8I8, 1, 8192, 28672, 16, 32, True),
                ("rhs_kn_s8_16x16", torch.int8, uk.PACK_TYPE_I8I8, 1, 16384, 16384, 16, 16, True),
                ("rhs_kn_s8_16x2", torch.int8, uk.PACK_TYPE_I8I8, 1, 16384, 16384, 16, 2, True),
                ("rhs_kn_bf16_16x2", torch.bfloat16, uk.PACK_TYPE_BF16BF16, 2, 8192, 16384, 16, 2, True),
                ("lhs_mk_s8_16x2", torch.int8, uk.PACK_TYPE_I8I8, 1, 16384, 16384, 16, 2, False),
            ]
            ops, keep = [], {"forms": []}
            lib = self.lib
            for i, (oname, dt, tf, es, rows, cols, X0, K0, kn) in enumerate(forms):
                if dt == torch.int8:
                    x = self.uniform_s8((rows, cols), 40 + i)
                else:
                    x = self.normal((rows, cols), dt, 40 + i)
                out = self.empty(rows * cols, dt)
                if kn:     # rows run along K, columns along N
                    flags = tf | uk.PACK_TRANSPOSE_INNER | uk.PACK_TRANSPOSE_OUTER
                    o0, o1 = cols // X0, rows // K0
                else:      # rows along M, columns along K
                    flags = tf
                    o0, o1 = rows // X0, cols // K0

                def launch(xp=x.data_ptr(), op_=out.data_ptr(), rows=rows, cols=cols, o0=o0, o1=o1,
                           X0=X0, K0=K0, flags=flags):
                    lib.pack(xp, 0, cols, 1, op_, 0, o1 * X0 * K0, X0 * K0, rows, cols, o0, o1, X0, K0,
                             0, flags)
                ops.append(Op(oname, launch, 0.0, float(2 * rows * cols * es), "hbm"))
                keep["forms"].append((oname, x, out, X0, K0, kn))
            return Workload(name, "pack of matmul operands that need an element-wise transposition: row-major "
                            "[K][N] right-hand sides (TRANSPOSE_INNER + TRANSPOSE_OUTER) and the 16x2 s8 tile",
                            ops, 0.0, sum(o.bytes for o in ops), "u8", keep)
        if name in ("c5_pack_f32_12288x12289", "c5_pack_f32_12289x12288"):
            rows, cols = (12288, 12289) if name.endswith("12289") else (12289, 12288)
            x = self.normal((rows, cols), torch.float32, 12)
            o0, o1 = -(-rows // 16), cols
            packed = self.empty(o0 * o1 * 16, torch.float32)
            back = self.empty(rows * cols, torch.float32)
            pad = 0xBF800000  # -1.0f
            ops = [self._pack_op("pack", x, rows, cols, packed, 16, 1, uk.PACK_TYPE_F32F32, 4,
                                 pad=pad, transpose_outer=True),
                   self._unpack_op("unpack", packed, back, rows, cols, 16, 1,
                                   uk.UNPACK_TYPE_F32F32, 4, transpose_outer=True)]
            return Workload(name, f"pack+unpack f32 {rows}x{cols} tiles 16x1 TRANSPOSE_OUTER pad -1.0",
                            ops, 0.0, sum(o.bytes for o in ops), "f32",
                            dict(x=x, packed=packed, back=back, rows=rows, cols=cols))
        raise KeyError(name)

    # ------------------------------------------------------------------ timing
    KIND = {"pack": 0, "unpack": 1, "mmt4d": 2, "conv": 3}

    def evict_cache(self):
        """Reads 1 GiB that nothing else uses (a torch reduction on the launch
        stream): afterwards the 256 MB memory-side cache holds none of the
        operands of earlier launches, and no modified lines either. Launches
        that rotate over three sets of buffers time the same (measured on pack:
        98.8 / 98.9, 91.6 / 91.2, 251 / 254 us)."""
        torch = self.torch
        if getattr(self, "_evict", None) is None:
            self._evict = torch.zeros(1 << 28, dtype=torch.int32, device="cuda")
        with torch.cuda.stream(self.stream):
            self._evict.max()

    def time_op(self, op: Op, iters: int, warmup: int = 5, cold: bool = False):
        """(average, minimum, median) device duration in microseconds of
        `iters` launches. Each launch carries its own HIP start/stop event pair
        on the launch stream (iree_uk_amd_timing_begin/end), which timestamps
        the kernel itself. `cold`: the memory-side cache is emptied of the
        operands before every timed launch (launches on the same buffers one
        after the other find up to 256 MB of them still there)."""
        torch = self.torch
        import time
        if op.external:
            with torch.cuda.stream(self.stream):
                for _ in range(warmup):
                    op.launch()
                evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                       for _ in range(iters)]
                for a, b in evs:
                    a.record(self.stream)
                    op.launch()
                    b.record(self.stream)
            self.stream.synchronize()
            us = [a.elapsed_time(b) * 1e3 for a, b in evs]
            return sum(us) / len(us), min(us), sorted(us)[len(us) // 2]
        with torch.cuda.stream(self.stream):
            # Same clock-settle phase as run_steps, then the warm-up launches.
            t_settle = time.perf_counter()
            while time.perf_counter() - t_settle < self.settle_seconds:
                for _ in range(4):
                    op.launch()
                self.stream.synchronize()
            for _ in range(warmup):
                op.launch()
            op.kernel = self.lib.last_kernel_name()
            self.stream.synchronize()
            self.lib.timing_begin()
            for _ in range(iters):
                if cold:
                    self.evict_cache()
                op.launch()
            recs = self.lib.timing_end()
        # A call may launch two kernels (whole K steps + remainder): sum per call.
        per_call = len(recs) // iters
        us = [sum(t for _, t in recs[i * per_call:(i + 1) * per_call]) for i in range(iters)]
        return sum(us) / len(us), min(us), sorted(us)[len(us) // 2]

    @staticmethod
    def roofline(op: Op, avg_us: float) -> dict:
        if op.bound in ("mfma", "vdot2"):
            achieved = op.flops / (avg_us * 1e-6) / 1e12
            peak = PEAK_TFLOPS[op.dtype]
            unit = "TFLOP/s"
        else:
            achieved = op.bytes / (avg_us * 1e-6) / 1e9
            peak = PEAK_HBM_GBPS
            unit = "GB/s"
        return {"bound": op.bound, "achieved": round(achieved, 3), "peak": peak,
                "unit": unit, "frac": round(achieved / peak, 4), "traffic": None}

    def run_steps(self, wl: Workload, steps: int, warmup: int, dominant: str):
        """Runs the whole workload `warmup` untimed times, then twice `steps`
        times, each pass bracketed by a synchronize on both sides and timed on
        the wall clock:
          pass 1, launches only: seconds per step of the whole job;
          pass 2, every launch carrying a HIP start/stop event pair on the
          launch stream: average device microseconds per launch of the
          dominant op (the event pairs serialize the queue a little, so this
          pass is slower as a whole and is reported separately).
        Returns (seconds per step, seconds per step with events, dominant us)."""
        import time
        torch = self.torch
        dom_kind = self.KIND["mmt4d" if dominant == "mmt4d" else
                             ("conv" if dominant == "conv" else
                              ("unpack" if dominant.startswith("unpack") else "pack"))]
        n_dom = sum(1 for op in wl.ops if op.name == dominant)
        with torch.cuda.stream(self.stream):
            # The device needs tens of milliseconds of load before its clocks
            # settle (the first ~60 steps of the f16 chain run ~12 % slower than
            # the following ones): run untimed steps for `settle_seconds` first.
            t_settle = time.perf_counter()
            while time.perf_counter() - t_settle < self.settle_seconds:
                for _ in range(8):
                    for op in wl.ops:
                        op.launch()
                torch.cuda.synchronize()
            for _ in range(warmup):
                for op in wl.ops:
                    op.launch()
            for op in wl.ops:
                op.launch()
                if not op.external:
                    op.kernel = self.lib.last_kernel_name()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                for op in wl.ops:
                    op.launch()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            self.lib.timing_begin()
            t2 = time.perf_counter()
            for _ in range(steps):
                for op in wl.ops:
                    op.launch()
            torch.cuda.synchronize()
            t3 = time.perf_counter()
            recs = self.lib.timing_end(capacity=max(4096, 8 * steps * len(wl.ops)))
        dom_total = sum(t for k, t in recs if k == dom_kind)
        # Ops of the same kind as the dominant one but with another name (e.g.
        # pack_lhs vs pack_rhs) only occur for pure data-movement workloads,
        # where the figure is then the average over that kind.
        n_kind = sum(1 for op in wl.ops if self.KIND.get(op.name.split("_")[0], -1) == dom_kind)
        dom_us = dom_total / (steps * max(1, n_kind if n_dom == 0 else n_kind)) if recs else math.nan
        return (t1 - t0) / steps, (t3 - t2) / steps, dom_us

    def shape_survey(self, reps: int = 15) -> str:
        """mmt4d on M x N x K problems shaped like a transformer's projections
        (M tokens from 256 to 4096 against five weight shapes), 16x16 tiles with
        16-byte tile rows, s8 / f16 / bf16: microseconds, fraction of the
        published peak and the kernel that ran, and beside each the GEMM that
        this image's PyTorch dispatches to the vendor library for the same
        problem on row-major operands (torch._int_mm / torch.matmul, B given as
        [N][K]) in the same process. The operands of the two differ in layout
        only; the comparison is context, not a baseline."""
        import time
        torch, lib = self.torch, self.lib

        def settle(f):
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.25:
                for _ in range(4):
                    f()
                torch.cuda.synchronize()

        def time_ours(f):
            with torch.cuda.stream(self.stream):
                settle(f)
                for _ in range(3):
                    f()
                name = lib.last_kernel_name()
                lib.timing_begin()
                for _ in range(reps):
                    f()
                recs = lib.timing_end()
            per = len(recs) // reps
            ts = sorted(sum(t for _, t in recs[i * per:(i + 1) * per]) for i in range(reps))
            return ts[len(ts) // 2], name

        def time_torch(f):
            settle(f)
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                   for _ in range(reps)]
            for a, b in evs:
                a.record()
                f()
                b.record()
            torch.cuda.synchronize()
            ts = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)
            return ts[len(ts) // 2]

        lines = ["type     M x N x K              ours us  frac  kernel                  vendor us  frac  ours/vendor"]
        ratios = {}
        for (tname, tflag, tdt, K0, peak) in (("s8", uk.MMT4D_TYPE_S8S8S32, torch.int8, 16, PEAK_TFLOPS["s8"]),
                                              ("f16", uk.MMT4D_TYPE_F16F16F32, torch.float16, 8, PEAK_TFLOPS["f16"]),
                                              ("bf16", uk.MMT4D_TYPE_BF16BF16F32, torch.bfloat16, 8, PEAK_TFLOPS["bf16"])):
            for (N, K) in ((4096, 4096), (14336, 4096), (4096, 14336), (28672, 8192), (8192, 8192)):
                for M in (256, 512, 1024, 2048, 4096):
                    M1, N1, K1 = M // 16, N // 16, K // K0
                    if tdt == torch.int8:
                        a = torch.randint(-128, 128, (M, K), device="cuda", dtype=tdt)
                        b = torch.randint(-128, 128, (N, K), device="cuda", dtype=tdt)
                    else:
                        a = torch.randn(M, K, device="cuda", dtype=tdt)
                        b = torch.randn(N, K, device="cuda", dtype=tdt)
                    out = torch.empty(M * N, device="cuda",
                                      dtype=torch.int32 if tdt == torch.int8 else torch.float32)
                    lp, rp, op_ = a.data_ptr(), b.data_ptr(), out.data_ptr()
                    # (the same bytes read as tiled operands: timing does not depend on the values' order)
                    us, kn = time_ours(lambda: lib.mmt4d(lp, 0, K1 * 16 * K0, rp, 0, K1 * 16 * K0, op_, 0,
                                                         N1 * 256, M1, N1, K1, 16, 16, K0, tflag))
                    bt = b.t()
                    try:
                        v = time_torch((lambda: torch._int_mm(a, bt)) if tdt == torch.int8
                                       else (lambda: torch.matmul(a, bt)))
                    except Exception:   # an op this build of torch does not have
                        v = float("nan")
                    fl = 2.0 * M * N * K
                    ratios.setdefault(tname, []).append(us / v)
                    lines.append(f"{tname:5s} {M:5d} x {N:5d} x {K:5d}  {us:9.1f}  {fl / us / 1e6 / peak:.3f}  "
                                 f"{kn.replace('mmt4d_mfma_', ''):22s} {v:9.1f}  {fl / v / 1e6 / peak:.3f}  {us / v:.2f}")
                    del a, b, bt, out
        for tname, r in ratios.items():
            r = sorted(x for x in r if x == x)
            if r:
                lines.append(f"{tname}: ours/vendor between {r[0]:.2f} and {r[-1]:.2f}, median {r[len(r) // 2]:.2f} "
                             f"over {len(r)} shapes")
        return "\n".join(lines)

    def tile_survey(self, size: int = 2048, reps: int = 5) -> str:
        """Every mmt4d type on the tile shapes the reference's own CPU kernels
        use (arch/x86_64/mmt4d_x86_64_tiles.inl, arch/arm_64/mmt4d_arm_64_tiles.inl
        and the s8 x s4 kernels of arch/arm_64/mmt4d_arm_64_*.c) at size^3:
        which kernel serves it, microseconds, operations per second. The 16-bit
        outputs run once as the reference defines them without
        SKIP_INTERMEDIATE_ROUNDINGS (a rounding per K tile, which only the
        scalar kernel reproduces) and once with the flag."""
        torch, lib = self.torch, self.lib
        skip = uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
        cases = [
            ("f32", uk.MMT4D_TYPE_F32F32F32, (32, 32, 32), [(16, 16, 1), (8, 8, 1), (8, 4, 1)]),
            ("f16 -> f32", uk.MMT4D_TYPE_F16F16F32, (16, 16, 32), [(16, 16, 1), (8, 8, 1)]),
            ("f16 -> f16", uk.MMT4D_TYPE_F16F16F16, (16, 16, 16), [(16, 16, 1), (8, 8, 1)]),
            ("f16 -> f16, skip", uk.MMT4D_TYPE_F16F16F16 | skip, (16, 16, 16), [(16, 16, 1), (8, 8, 1)]),
            ("bf16 -> f32", uk.MMT4D_TYPE_BF16BF16F32, (16, 16, 32), [(16, 16, 2), (8, 8, 4)]),
            ("bf16 -> bf16", uk.MMT4D_TYPE_BF16BF16BF16, (16, 16, 16), [(16, 16, 2), (8, 8, 4)]),
            ("bf16 -> bf16, skip", uk.MMT4D_TYPE_BF16BF16BF16 | skip, (16, 16, 16), [(16, 16, 2), (8, 8, 4)]),
            ("s8", uk.MMT4D_TYPE_S8S8S32, (8, 8, 32), [(16, 16, 2), (8, 8, 1), (8, 8, 4), (8, 8, 8)]),
            ("s16 x s16", uk.MMT4D_TYPE_S16S16S32, (16, 16, 32), [(16, 16, 2), (8, 8, 1)]),
            ("s16 x s8", uk.MMT4D_TYPE_S16S8S32, (16, 8, 32), [(16, 16, 2)]),
            ("s16 x u4", uk.MMT4D_TYPE_S16U4S32, (16, 4, 32), [(1, 32, 8)]),
            ("s8 x s4", uk.MMT4D_TYPE_S8S4S32, (8, 4, 32), [(4, 16, 2), (8, 8, 8), (4, 8, 16), (1, 8, 16)]),
        ]
        S = size
        lines = [f"mmt4d {S}^3 on the reference's CPU tile shapes",
                 "type                 M0xN0xK0          us      TOP/s  kernel"]
        for nm, tf, bits, tiles in cases:
            for (M0, N0, K0) in tiles:
                M1, N1, K1 = S // M0, S // N0, S // K0
                # small byte values: finite in every float type, and timing does not depend on them
                a = torch.randint(0, 40, (S * S * bits[0] // 8,), device="cuda", dtype=torch.uint8)
                b = torch.randint(0, 40, (S * S * bits[1] // 8,), device="cuda", dtype=torch.uint8)
                out = torch.empty(S * S * bits[2] // 8, device="cuda", dtype=torch.uint8)
                ap, bp, op_ = a.data_ptr(), b.data_ptr(), out.data_ptr()
                flags = tf | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION

                def f():
                    lib.mmt4d(ap, 0, K1 * M0 * K0, bp, 0, K1 * N0 * K0, op_, 0, N1 * M0 * N0,
                              M1, N1, K1, M0, N0, K0, flags)
                with torch.cuda.stream(self.stream):
                    for _ in range(2):
                        f()
                    name = lib.last_kernel_name()
                    lib.timing_begin()
                    for _ in range(reps):
                        f()
                    recs = lib.timing_end()
                per = len(recs) // reps
                ts = sorted(sum(t for _, t in recs[i * per:(i + 1) * per]) for i in range(reps))
                us = ts[len(ts) // 2]
                lines.append(f"{nm:20s} {M0:2d}x{N0:2d}x{K0:2d}  {us:10.1f}  {2.0 * S ** 3 / us / 1e6:9.1f}  {name}")
                del a, b, out
        return "\n".join(lines)

    def k_sweep(self, name: str, variants=(0, 16, 8, 1), reps: int = 15) -> str:
        """T(K) of the mmt4d op of a square workload (`<type>_mmt4d_<size>_k<K0>`)
        under forced kernel variants, K from 1/16 of the workload's K up to all
        of it (the same M x N output every time, the operands' first K tiles of
        every panel), variants interleaved launch by launch so that clock drift
        hits them alike. A straight-line fit gives what a launch costs apart
        from its K loop (launch, pipeline fill, the output's way out) and what
        1024 more bytes of K per row cost. One more row runs the full K with all
        panels aliased onto the first one (panel strides of zero: every workgroup
        reads the same rows, so the operands never leave the caches): what the
        kernel does when the memory system beyond the L2 costs nothing. Returns
        the table as text."""
        torch = self.torch
        wl = self.workload(name)
        op = next(o for o in wl.ops if o.name == "mmt4d")
        k = wl.keep
        M1, N1, K1, M0, N0, K0 = (k[x] for x in ("M1", "N1", "K1", "M0", "N0", "K0"))
        tf = self.MMT4D_TYPE[op.dtype]
        lib = self.lib
        lp, rp, outp = k["lhs4"].data_ptr(), k["rhs4"].data_ptr(), k["out4"].data_ptr()
        es = k["lhs4"].element_size()
        ks = [K1 >> s for s in (4, 3, 2, 1, 0) if (K1 >> s) * K0 * es >= 256]

        def call(variant, kt, alias):
            lib.set_kernel_mode(uk.KERNEL_MODE_MFMA_VARIANT + variant if variant else uk.KERNEL_MODE_AUTO)
            lib.mmt4d(lp, 0, 0 if alias else K1 * M0 * K0, rp, 0, 0 if alias else K1 * N0 * K0, outp, 0,
                      N1 * M0 * N0, M1, N1, kt, M0, N0, K0, tf)

        cases = [(v, kt, False) for v in variants for kt in ks] + [(v, K1, True) for v in variants]
        times = {c: [] for c in cases}
        names = {}
        with torch.cuda.stream(self.stream):
            for c in cases:
                call(*c)
                names[c[0]] = lib.last_kernel_name()
            for _ in range(3):
                for c in cases:
                    call(*c)
            lib.synchronize()
            for _ in range(reps):
                for c in cases:
                    lib.timing_begin()
                    call(*c)
                    times[c].append(sum(t for _, t in lib.timing_end()))
        lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
        med = {c: sorted(t)[len(t) // 2] for c, t in times.items()}
        peak = PEAK_TFLOPS[op.dtype]
        kb = [kt * K0 * es for kt in ks]   # bytes of K per row
        lines = [f"T(K) of the mmt4d op of {name} ({wl.description}): median of {reps} launches in us, variants "
                 "interleaved launch by launch.",
                 "K is given in bytes per tile row panel; `fit` is the straight line through the two longest "
                 "K: us at K = 0, us per 1024 bytes of K.",
                 "`cached operands`: all of K with every panel aliased onto the first (panel strides 0).", ""]
        head = "%-4s %-34s" % ("v", "kernel") + "".join("%10d" % b for b in kb) + "   fit: const   /1024 B   frac@full   cached operands"
        lines.append(head)
        for v in variants:
            row = [med[(v, kt, False)] for kt in ks]
            slope = (row[-1] - row[-2]) / (kb[-1] - kb[-2]) * 1024
            const = row[-1] - slope * kb[-1] / 1024
            frac = op.flops / (row[-1] * 1e-6) / 1e12 / peak
            lines.append("%-4d %-34s" % (v, names[v]) + "".join("%10.1f" % t for t in row) +
                         "   %10.1f %9.2f %11.3f %18.1f" % (const, slope, frac, med[(v, K1, True)]))
        return "\n".join(lines) + "\n"

    MMT4D_TYPE = {"s8": uk.MMT4D_TYPE_S8S8S32, "f16": uk.MMT4D_TYPE_F16F16F32,
                  "bf16": uk.MMT4D_TYPE_BF16BF16F32, "f32": uk.MMT4D_TYPE_F32F32F32,
                  "f8": uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32}

    def measured_mfma_peak(self, dtype: str, zeros: bool = False, seconds: float = 0.02) -> float:
        """TOP/s (TFLOP/s) of a loop of nothing but this type's MFMA
        instruction with the mmt4d kernels' register blocking, 8 waves per CU,
        register operands taken from random bytes of the type's value range (or
        zeros): the ceiling the matrix cores hold on this device at the clock
        its power limit allows, before a single operand is moved. Runs about
        `seconds` after a settle phase of the same loop."""
        torch = self.torch
        n = 1 << 16
        if zeros:
            operands = torch.zeros(n, dtype=torch.uint8, device="cuda")
        elif dtype == "s8":
            operands = self.uniform_s8((n,), 901).view(torch.uint8)
        elif dtype == "f8":
            operands = self.normal_f8((n,), 902)
        elif dtype == "f32":
            operands = self.normal((n // 4,), torch.float32, 903).view(torch.uint8)
        else:
            operands = self.normal((n // 2,), torch.float16 if dtype == "f16" else torch.bfloat16,
                                   904).view(torch.uint8)
        sink = torch.zeros(4 * 512 * 1024, dtype=torch.int32, device="cuda")
        st = self.stream.cuda_stream
        tf = self.MMT4D_TYPE[dtype]
        self.stream.synchronize()
        # Size the loop from a short run, then let the clocks settle under it.
        rate = self.lib.probe_mfma_peak(tf, operands.data_ptr(), n, 2000, sink.data_ptr(), st)
        per_iter = 2.0 * 16 * 16 * {"s8": 64, "f8": 128, "f32": 16}.get(dtype, 32) * 32 * 8 * 512
        iters = max(1000, int(rate * seconds / per_iter))
        best = 0.0
        for _ in range(4):
            best = max(best, self.lib.probe_mfma_peak(tf, operands.data_ptr(), n, iters,
                                                      sink.data_ptr(), st))
        # A loop of nothing but MFMAs cannot beat the published peak and, on a
        # healthy part, does not fall far below it: anything else means the probe
        # did not measure what it is meant to (e.g. its loop was optimized away).
        peak = PEAK_TFLOPS[dtype] * 1e12
        if not 0.3 * peak <= best <= 1.02 * peak:
            raise RuntimeError(f"MFMA-only probe for {dtype} reads {best / 1e12:.1f} T/s against a "
                               f"published peak of {peak / 1e12:.1f}: not a valid ceiling")
        return best / 1e12

    def measured_mfma_waves(self, zeros: bool, seconds: float = 0.02) -> dict:
        """TOP/s of the s8 MFMA-only loop (MFMAs as assembly) with one and with
        two waves on every SIMD (one workgroup per CU): a lone wave keeps the
        matrix pipe as full as two do. On all-zero operands the comparison is
        free of the power limit."""
        torch = self.torch
        n = 1 << 16
        operands = (torch.zeros(n, dtype=torch.uint8, device="cuda") if zeros
                    else self.uniform_s8((n,), 901).view(torch.uint8))
        sink = torch.zeros(4 * 512 * 1024, dtype=torch.int32, device="cuda")
        st = self.stream.cuda_stream
        self.stream.synchronize()
        out = {}
        for waves in (2, 1):
            rate = self.lib.probe_mfma_peak_waves(operands.data_ptr(), n, 2000, waves, sink.data_ptr(), st)
            per_iter = 2.0 * 16 * 16 * 64 * 32 * (4 * waves) * 256
            iters = max(1000, int(rate * seconds / per_iter))
            best = 0.0
            for _ in range(4):
                best = max(best, self.lib.probe_mfma_peak_waves(operands.data_ptr(), n, iters, waves,
                                                                sink.data_ptr(), st))
            out[waves] = best / 1e12
        return out

    def copy2d_ceiling_gbps(self, rows: int, row_bytes: int, src_pitch: int, dst_pitch: int,
                            iters: int = 10, cold: bool = False) -> float:
        """GB/s (read + write) of a plain copy of rows x row_bytes between the
        two pitches: what a pack / unpack of that matrix could reach if the
        transposition were free. `cold`: as many times the rows as make each
        side 3 GB or more, so that what one launch leaves in the 256 MB
        memory-side cache is a small part of what the next one moves."""
        torch = self.torch
        if cold:
            rows *= max(1, -(-(3 << 30) // (rows * row_bytes)))
        src = torch.empty(rows * src_pitch, dtype=torch.uint8, device="cuda")
        dst = torch.empty(rows * dst_pitch, dtype=torch.uint8, device="cuda")
        self.stream.synchronize()
        sec, per = self.lib.probe_copy2d_variants(src.data_ptr(), src_pitch, dst.data_ptr(), dst_pitch,
                                                  row_bytes, rows, iters, self.stream.cuda_stream)
        # (the last variant writes whole 128-byte lines only, whatever the pitch)
        self.last_copy2d_whole_lines_gbps = 2.0 * rows * row_bytes / per[4] / 1e9
        return 2.0 * rows * row_bytes / sec / 1e9

    def measured_copy_gbps(self, nbytes: int = 1 << 30, iters: int = 10) -> float:
        """Device-to-device copy rate (read + write bytes), for a measured HBM
        ceiling next to the nominal one."""
        torch = self.torch
        a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        b = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        with torch.cuda.stream(self.stream):
            b.copy_(a)
            s = torch.cuda.Event(enable_timing=True)
            e = torch.cuda.Event(enable_timing=True)
            s.record(self.stream)
            for _ in range(iters):
                b.copy_(a)
            e.record(self.stream)
        self.stream.synchronize()
        return 2.0 * nbytes * iters / (s.elapsed_time(e) * 1e-3) / 1e9
