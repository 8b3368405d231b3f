"""ctypes access to the CPU checkers for pack / mmt4d / unpack.

TEST INFRASTRUCTURE, NOT PRODUCT CODE: only tests, the smoke check and the
benchmark's cpu_baseline leg import this module. The shipped package
(``iree_amd``) never does.

Two checkers share one calling convention (the argument lists of the reference
entry points, runtime/src/iree/builtins/ukernel/{mmt4d.h:14-21, pack.h:26-34,
unpack.h:17-25}):

* ``Checker("oracle")`` -- ``oracle/liboracle_uk.so``, our scalar C restatement
  (``oracle/uk_oracle.c``); always available (built with gcc on first use).
* ``Checker("reference")`` -- ``oracle/_ref/libiree_uk_ref.so``, the unmodified
  reference C ukernels compiled by ``oracle/Makefile``; present only where it
  was built (it travels to the GPU box as a prebuilt file).

All buffers are numpy arrays; offsets/strides are in elements.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import threading
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle_uk.so")
REF_SO = os.path.join(_HERE, "_ref", "libiree_uk_ref.so")

_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_u32 = ctypes.c_uint32
_u64 = ctypes.c_uint64
_vp = ctypes.c_void_p

_MMT4D_ARGS = [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64,
               _i64, _i32, _i32, _i32, _u32, _vp]
_PACK_ARGS = [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
              _i64, _i64, _i64, _u64, _u32, _vp]
_UNPACK_ARGS = [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                _i64, _i64, _i64, _u32, _vp]
_CONV_ARGS = ([_vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64,
               _i64] + [_i64] * 7 + [_i32] * 4 + [_u32, _vp])

# Bit positions of cpu_data[0] on x86-64
# (runtime/src/iree/schemas/cpu_feature_bits.inl:85-117), keyed by the
# /proc/cpuinfo flag that reports the feature.
_X86_BITS = {
    "avx": 10, "fma": 11, "f16c": 14, "avx2": 15, "avx512f": 20,
    "avx512cd": 21, "avx512vl": 22, "avx512dq": 23, "avx512bw": 24,
    "avx512_vnni": 28, "avx512_bf16": 31,
}


def build_oracle() -> str:
    """Compiles oracle/uk_oracle.c (and, where the reference checkout exists,
    oracle/_ref) with the committed Makefile."""
    subprocess.run(["make", "-C", _HERE, "-j8", "all"], check=True,
                   stdout=subprocess.DEVNULL)
    return ORACLE_SO


def host_cpu_data(enable: bool = True) -> np.ndarray:
    """The 8-word cpu_data array (runtime/src/iree/schemas/cpu_data.h:63) for
    this host; all zeros (= generic code paths only) when enable is False."""
    words = np.zeros(8, dtype=np.uint64)
    if not enable:
        return words
    flags: set[str] = set()
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    flags = set(line.split(":", 1)[1].split())
                    break
    except OSError:
        pass
    v = 0
    for name, bit in _X86_BITS.items():
        if name in flags:
            v |= 1 << bit
    words[0] = v
    return words


def _ptr(a: np.ndarray | None, byte_shift: int = 0):
    if a is None:
        return None
    return ctypes.c_void_p(a.ctypes.data + byte_shift)


class Checker:
    def __init__(self, kind: str = "oracle"):
        self.kind = kind
        if kind == "oracle":
            if not os.path.exists(ORACLE_SO):
                build_oracle()
            self.lib = ctypes.CDLL(ORACLE_SO)
            names = ("uk_oracle_mmt4d", "uk_oracle_pack", "uk_oracle_unpack")
            restype = ctypes.c_int
        elif kind == "reference":
            if not os.path.exists(REF_SO):
                raise FileNotFoundError(REF_SO)
            self.lib = ctypes.CDLL(REF_SO)
            names = ("iree_uk_mmt4d", "iree_uk_pack", "iree_uk_unpack")
            restype = None
        else:
            raise ValueError(kind)
        self._mmt4d = getattr(self.lib, names[0])
        self._pack = getattr(self.lib, names[1])
        self._unpack = getattr(self.lib, names[2])
        self._conv = getattr(self.lib, "uk_oracle_conv_nchwc" if kind == "oracle"
                             else "iree_uk_conv_nchwc")
        for fn, args in ((self._mmt4d, _MMT4D_ARGS), (self._pack, _PACK_ARGS),
                         (self._unpack, _UNPACK_ARGS), (self._conv, _CONV_ARGS)):
            fn.argtypes = args
            fn.restype = restype
        if kind == "oracle":
            self.lib.uk_oracle_f8e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
            self.lib.uk_oracle_f8e4m3fn_to_f32.restype = ctypes.c_float
            self.lib.uk_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
            self.lib.uk_oracle_f16_to_f32.restype = ctypes.c_float
            self.lib.uk_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
            self.lib.uk_oracle_bf16_to_f32.restype = ctypes.c_float
            self.lib.uk_oracle_f32_to_f16.argtypes = [ctypes.c_float]
            self.lib.uk_oracle_f32_to_f16.restype = ctypes.c_uint16
            self.lib.uk_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
            self.lib.uk_oracle_f32_to_bf16.restype = ctypes.c_uint16
            self.lib.uk_oracle_set_flush_subnormal_inputs.argtypes = [ctypes.c_int]
        # The reference reads cpu_data[0] unconditionally on x86-64.
        self.cpu_data = host_cpu_data(enable=False)

    @staticmethod
    def reference_available() -> bool:
        return os.path.exists(REF_SO)

    def use_host_cpu_features(self, enable: bool = True):
        """Lets the reference pick its AVX2/AVX-512 tile functions (no effect on
        the oracle, which has one scalar code path)."""
        self.cpu_data = host_cpu_data(enable)
        return self

    # -- raw entry points (same positional arguments as the reference) -------
    def mmt4d(self, lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0,
              out, out_offset, out_stride0, M, N, K, M0, N0, K0, flags,
              lhs_shift=0, rhs_shift=0, out_shift=0):
        """lhs/rhs/out are numpy arrays; *_shift is a byte displacement added to
        the array's base address (negative to emulate `buffer - offset`)."""
        r = self._mmt4d(_ptr(lhs, lhs_shift), lhs_offset, lhs_stride0,
                        _ptr(rhs, rhs_shift), rhs_offset, rhs_stride0,
                        _ptr(out, out_shift), out_offset, out_stride0, M, N, K,
                        M0, N0, K0, flags, _ptr(self.cpu_data))
        if self.kind == "oracle" and r != 0:
            raise ValueError(f"oracle mmt4d rejected flags {flags:#x}")

    def pack(self, inp, in_offset, in_stride0, in_stride1, out, out_offset,
             out_stride0, out_stride1, in_size0, in_size1, out_size0, out_size1,
             out_size2, out_size3, padding_value, flags, in_shift=0,
             out_shift=0):
        r = self._pack(_ptr(inp, in_shift), in_offset, in_stride0, in_stride1,
                       _ptr(out, out_shift), out_offset, out_stride0,
                       out_stride1, in_size0, in_size1, out_size0, out_size1,
                       out_size2, out_size3, padding_value, flags,
                       _ptr(self.cpu_data))
        if self.kind == "oracle" and r != 0:
            raise ValueError(f"oracle pack rejected flags {flags:#x}")

    def unpack(self, inp, in_offset, in_stride0, in_stride1, out, out_offset,
               out_stride0, out_stride1, in_size0, in_size1, in_size2, in_size3,
               out_size0, out_size1, flags, in_shift=0, out_shift=0):
        r = self._unpack(_ptr(inp, in_shift), in_offset, in_stride0, in_stride1,
                         _ptr(out, out_shift), out_offset, out_stride0,
                         out_stride1, in_size0, in_size1, in_size2, in_size3,
                         out_size0, out_size1, flags, _ptr(self.cpu_data))
        if self.kind == "oracle" and r != 0:
            raise ValueError(f"oracle unpack rejected flags {flags:#x}")

    def conv_nchwc(self, inp, input_offset, input_stride_n, input_stride_ic_outer,
                   input_stride_h, flt, filter_offset, filter_stride_oc_outer,
                   filter_stride_ic_outer, filter_stride_fh, out, output_offset,
                   output_stride_n, output_stride_oc_outer, output_stride_oh, N, OC_outer, OH,
                   OW, IC_outer, FH, FW, k0, c0, stride_h, stride_w, flags, in_shift=0,
                   filter_shift=0, out_shift=0):
        """Positional arguments of iree_uk_conv_nchwc
        (runtime/src/iree/builtins/ukernel/conv_nchwc.h:14-27)."""
        r = self._conv(_ptr(inp, in_shift), input_offset, input_stride_n, input_stride_ic_outer,
                       input_stride_h, _ptr(flt, filter_shift), filter_offset,
                       filter_stride_oc_outer, filter_stride_ic_outer, filter_stride_fh,
                       _ptr(out, out_shift), output_offset, output_stride_n,
                       output_stride_oc_outer, output_stride_oh, N, OC_outer, OH, OW, IC_outer,
                       FH, FW, k0, c0, stride_h, stride_w, flags, _ptr(self.cpu_data))
        if self.kind == "oracle" and r != 0:
            raise ValueError(f"oracle conv_nchwc rejected flags {flags:#x}")

    # -- threaded mmt4d: slabs of M (or N when M is small) through the
    # offset/stride parameters, the way IREE's task system slices work -------
    def mmt4d_threaded(self, threads, lhs, lhs_stride0, rhs, rhs_stride0, out,
                       out_stride0, M, N, K, M0, N0, K0, flags):
        threads = max(1, int(threads))
        jobs = []
        if M >= threads or M >= N:
            step = -(-M // threads)
            for m0 in range(0, M, step):
                m1 = min(M, m0 + step)
                jobs.append((m0 * lhs_stride0, 0, m0 * out_stride0, m1 - m0, N))
        else:
            step = -(-N // threads)
            for n0 in range(0, N, step):
                n1 = min(N, n0 + step)
                jobs.append((0, n0 * rhs_stride0, n0 * M0 * N0, M, n1 - n0))

        def run(job):
            lo, ro, oo, m, n = job
            self.mmt4d(lhs, lo, lhs_stride0, rhs, ro, rhs_stride0, out, oo,
                       out_stride0, m, n, K, M0, N0, K0, flags)

        if len(jobs) == 1:
            run(jobs[0])
        else:
            with ThreadPoolExecutor(max_workers=len(jobs)) as ex:
                list(ex.map(run, jobs))
        return len(jobs)

    # -- scalar helpers (oracle only) ----------------------------------------
    def f8e4m3fn_to_f32(self, v: int) -> float:
        return float(self.lib.uk_oracle_f8e4m3fn_to_f32(v))


_lock = threading.Lock()
_cache: dict[str, Checker] = {}


def get(kind: str = "oracle") -> Checker:
    with _lock:
        if kind not in _cache:
            _cache[kind] = Checker(kind)
        return _cache[kind]
