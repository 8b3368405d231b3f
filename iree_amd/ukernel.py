"""ctypes binding of libiree_uk_amd.so: the gfx950 pack / mmt4d / unpack ukernels.

The functions keep the names, positional argument order and meaning of the
reference C entry points (runtime/src/iree/builtins/ukernel/mmt4d.h:14-21,
pack.h:26-34, unpack.h:17-25); buffers are passed as integer addresses
(``tensor.data_ptr()`` of a device tensor, or a host address), offsets and
strides in elements.

There is no fallback: if the shared library has not been built, importing the
binding raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libiree_uk_amd.so")

# --- flag values (runtime/src/iree/builtins/ukernel/exported_bits.h:29-83) ---
MMT4D_TYPE_F32F32F32 = 0x01
MMT4D_TYPE_S8S8S32 = 0x02
MMT4D_TYPE_F16F16F32 = 0x03
MMT4D_TYPE_F16F16F16 = 0x04
MMT4D_TYPE_BF16BF16F32 = 0x05
MMT4D_TYPE_BF16BF16BF16 = 0x06
MMT4D_TYPE_S16S16S32 = 0x07
MMT4D_TYPE_S16U4S32 = 0x08
MMT4D_TYPE_S16S8S32 = 0x09
MMT4D_TYPE_S8S4S32 = 0x0A
MMT4D_TYPE_F8E4M3FNF8E4M3FNF32 = 0x80  # extension of this library
MMT4D_ACCUMULATE = 0x100
MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION = 0x200
MMT4D_SKIP_INTERMEDIATE_ROUNDINGS = 0x400
MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION = 0x1

PACK_TYPE_F32F32 = 0x01
PACK_TYPE_I8I8 = 0x02
PACK_TYPE_I32I32 = 0x03
PACK_TYPE_F16F16 = 0x04
PACK_TYPE_BF16BF16 = 0x05
PACK_TRANSPOSE_INNER = 0x100
PACK_TRANSPOSE_OUTER = 0x200

UNPACK_TYPE_F32F32 = 0x01
UNPACK_TYPE_I32I32 = 0x03
UNPACK_TYPE_F16F16 = 0x04
UNPACK_TYPE_BF16BF16 = 0x05
UNPACK_TRANSPOSE_INNER = 0x100
UNPACK_TRANSPOSE_OUTER = 0x200

POINTER_MODE_AUTO = 0
POINTER_MODE_DEVICE = 1
KERNEL_MODE_AUTO = 0
KERNEL_MODE_GENERIC = 1
KERNEL_MODE_MFMA_VARIANT = 16  # + 1..10: force an mmt4d MFMA workgroup shape

# (lhs bits, rhs bits, out bits) per mmt4d type value.
MMT4D_TYPE_BITS = {
    MMT4D_TYPE_F32F32F32: (32, 32, 32),
    MMT4D_TYPE_S8S8S32: (8, 8, 32),
    MMT4D_TYPE_F16F16F32: (16, 16, 32),
    MMT4D_TYPE_F16F16F16: (16, 16, 16),
    MMT4D_TYPE_BF16BF16F32: (16, 16, 32),
    MMT4D_TYPE_BF16BF16BF16: (16, 16, 16),
    MMT4D_TYPE_S16S16S32: (16, 16, 32),
    MMT4D_TYPE_S16U4S32: (16, 4, 32),
    MMT4D_TYPE_S16S8S32: (16, 8, 32),
    MMT4D_TYPE_S8S4S32: (8, 4, 32),
    MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: (8, 8, 32),
}
PACK_TYPE_BYTES = {PACK_TYPE_F32F32: 4, PACK_TYPE_I8I8: 1, PACK_TYPE_I32I32: 4,
                   PACK_TYPE_F16F16: 2, PACK_TYPE_BF16BF16: 2}

_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_u32 = ctypes.c_uint32
_u64 = ctypes.c_uint64
_vp = ctypes.c_void_p

STATUS_SCRATCH_TOO_SMALL = 100001
STATUS_NEEDS_ALLOCATION = 100002


class Mmt4dParams(ctypes.Structure):
    """iree_uk_mmt4d_params_t (include/iree_uk_amd.h; field order of
    runtime/src/iree/builtins/ukernel/mmt4d_internal.h:14-32)."""
    _fields_ = [("lhs_buffer", _vp), ("lhs_offset", _i64), ("lhs_stride0", _i64),
                ("rhs_buffer", _vp), ("rhs_offset", _i64), ("rhs_stride0", _i64),
                ("out_buffer", _vp), ("out_offset", _i64), ("out_stride0", _i64),
                ("M", _i64), ("N", _i64), ("K", _i64), ("M0", _i32), ("N0", _i32),
                ("K0", _i32), ("flags", _u32), ("cpu_data", _vp)]


ASSERT_HANDLER = ctypes.CFUNCTYPE(None, ctypes.c_char_p, ctypes.c_int,
                                  ctypes.c_char_p, ctypes.c_char_p)


class ContractViolation(RuntimeError):
    """Raised by the Python-side assert handler (see raise_on_violation)."""


def _share_hip_runtime_with_torch():
    """A process must hold ONE HIP runtime, or device pointers made by one copy
    are unknown to the other. PyTorch wheels bundle their own libamdhip64.so
    (soname libamdhip64.so.7) and load it by file name, so it has to be in the
    process before this library's NEEDED entry of the same soname is resolved;
    then both share it. Without PyTorch the system runtime is used."""
    import importlib.util
    import sys
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.origin:
        return
    libdir = os.path.join(os.path.dirname(spec.origin), "lib")
    for name in ("libhsa-runtime64.so", "libamdhip64.so"):
        cand = os.path.join(libdir, name)
        if os.path.exists(cand):
            try:
                ctypes.CDLL(cand, mode=ctypes.RTLD_GLOBAL)
            except OSError:
                return


class UKernelLibrary:
    """The loaded shared library with typed entry points."""

    def __init__(self, path: str = LIB_PATH):
        if not os.path.exists(path):
            raise ImportError(
                f"{path} is missing: build it with `python -m iree_amd.build` "
                "(there is no CPU or PyTorch fallback for these kernels)")
        self.path = path
        _share_hip_runtime_with_torch()
        self.lib = ctypes.CDLL(path)
        L = self.lib
        L.iree_uk_mmt4d.argtypes = [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64,
                                    _i64, _i64, _i64, _i64, _i32, _i32, _i32,
                                    _u32, _vp]
        L.iree_uk_mmt4d.restype = None
        L.iree_uk_mmt4d_info.argtypes = [_i32, _i32, _i32, _u32, _vp]
        L.iree_uk_mmt4d_info.restype = _u32
        L.iree_uk_pack.argtypes = [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64,
                                   _i64, _i64, _i64, _i64, _i64, _i64, _u64,
                                   _u32, _vp]
        L.iree_uk_pack.restype = None
        L.iree_uk_unpack.argtypes = [_vp, _i64, _i64, _i64, _vp, _i64, _i64,
                                     _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                     _u32, _vp]
        L.iree_uk_unpack.restype = None
        L.iree_uk_amd_mmt4d_unpack.argtypes = [_vp, _i64, _i64, _vp, _i64, _i64, _vp,
                                               _i64, _i64, _i64, _i64, _i64, _i64,
                                               _i64, _i32, _i32, _i32, _u32, _vp]
        L.iree_uk_amd_mmt4d_unpack.restype = None
        L.iree_uk_amd_mmt4d_dequant_unpack.argtypes = (
            [_vp, _i64, _i64] * 4 + [_i64, _i64, _vp, _vp, _i64, _i64, _i64,
                                     _i32, _i32, _i32, _u32, _vp])
        L.iree_uk_amd_mmt4d_dequant_unpack.restype = None
        L.iree_uk_conv_nchwc.argtypes = ([_vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64,
                                          _vp, _i64, _i64, _i64, _i64] + [_i64] * 7 +
                                         [_i32] * 4 + [_u32, _vp])
        L.iree_uk_conv_nchwc.restype = None
        L.iree_uk_amd_last_status.restype = ctypes.c_int
        L.iree_uk_amd_last_status_string.restype = ctypes.c_char_p
        L.iree_uk_amd_last_kernel_name.restype = ctypes.c_char_p
        L.iree_uk_amd_set_stream.argtypes = [_vp]
        L.iree_uk_amd_get_stream.restype = _vp
        L.iree_uk_amd_synchronize.restype = ctypes.c_int
        L.iree_uk_amd_set_pointer_mode.argtypes = [ctypes.c_int]
        L.iree_uk_amd_set_kernel_mode.argtypes = [ctypes.c_int]
        L.iree_uk_amd_set_persistent_workgroups.argtypes = [ctypes.c_int]
        L.iree_uk_amd_set_persistent_workgroups.restype = None
        L.iree_uk_amd_device_count.restype = ctypes.c_int
        L.iree_uk_amd_mmt4d_no_alloc.argtypes = [_vp]
        L.iree_uk_amd_mmt4d_no_alloc.restype = None
        L.iree_uk_amd_no_alloc_scratch_bytes.restype = _i64
        L.iree_uk_amd_set_k_slices.argtypes = [ctypes.c_int]
        L.iree_uk_amd_set_k_slices.restype = None
        L.iree_uk_amd_set_streamed_weights.argtypes = [ctypes.c_int]
        L.iree_uk_amd_set_streamed_weights.restype = None
        L.iree_uk_amd_last_k_slices.restype = ctypes.c_int
        L.iree_uk_amd_mfma_decline_count.restype = ctypes.c_uint64
        L.iree_uk_amd_version.restype = ctypes.c_char_p
        L.iree_uk_amd_set_assert_handler.argtypes = [_vp]
        L.iree_uk_amd_timing_begin.restype = None
        L.iree_uk_amd_staging_bytes.restype = _i64
        L.iree_uk_amd_device_alloc_count.restype = _i64
        L.iree_uk_amd_release_staging.restype = ctypes.c_int
        L.iree_uk_amd_workspace_bytes.restype = _i64
        L.iree_uk_amd_release_workspaces.restype = ctypes.c_int
        L.iree_uk_amd_timing_end.argtypes = [_vp, _vp, ctypes.c_int]
        L.iree_uk_amd_timing_end.restype = ctypes.c_int
        L.iree_uk_amd_probe_mfma_peak.argtypes = [_u32, _vp, _i64, ctypes.c_int, ctypes.c_int, _vp,
                                                  _vp, ctypes.POINTER(ctypes.c_double)]
        L.iree_uk_amd_probe_mfma_peak.restype = ctypes.c_int
        L.iree_uk_amd_probe_mfma_peak_waves.argtypes = [_vp, _i64, ctypes.c_int, ctypes.c_int, _vp, _vp,
                                                        ctypes.POINTER(ctypes.c_double)]
        L.iree_uk_amd_probe_mfma_peak_waves.restype = ctypes.c_int
        L.iree_uk_amd_probe_copy2d.argtypes = [_vp, _i64, _vp, _i64, _i64, _i64, ctypes.c_int, _vp,
                                               ctypes.POINTER(ctypes.c_double)]
        L.iree_uk_amd_probe_copy2d.restype = ctypes.c_int
        L.iree_uk_amd_probe_copy2d_variants.argtypes = [_vp, _i64, _vp, _i64, _i64, _i64, ctypes.c_int, _vp,
                                                        ctypes.POINTER(ctypes.c_double),
                                                        ctypes.POINTER(ctypes.c_double)]
        L.iree_uk_amd_probe_copy2d_variants.restype = ctypes.c_int
        L.iree_uk_amd_probe_ds_read_tr16.argtypes = [_vp, _vp, ctypes.c_int, _vp]
        L.iree_uk_amd_probe_ds_read_tr16.restype = ctypes.c_int
        self._handler_ref = None
        self._violations: list[str] = []

    # ----------------------------------------------------------------- entry
    def mmt4d(self, lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0,
              out, out_offset, out_stride0, M, N, K, M0, N0, K0, flags,
              cpu_data=None):
        self.lib.iree_uk_mmt4d(lhs, lhs_offset, lhs_stride0, rhs, rhs_offset,
                               rhs_stride0, out, out_offset, out_stride0, M, N,
                               K, M0, N0, K0, flags, cpu_data)
        self._check()

    def mmt4d_no_alloc(self, lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0,
                       out, out_offset, out_stride0, M, N, K, M0, N0, K0, flags, check=True):
        """iree_uk_amd_mmt4d_no_alloc: same arguments as mmt4d, passed as the
        params struct. With check=False the status is left for the caller to
        read (last_status) instead of being raised."""
        p = Mmt4dParams(lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0, out,
                        out_offset, out_stride0, M, N, K, M0, N0, K0, flags, None)
        self.lib.iree_uk_amd_mmt4d_no_alloc(ctypes.byref(p))
        if check:
            self._check()

    def last_status(self) -> int:
        return int(self.lib.iree_uk_amd_last_status())

    def last_status_string(self) -> str:
        return self.lib.iree_uk_amd_last_status_string().decode()

    def no_alloc_scratch_bytes(self) -> int:
        return int(self.lib.iree_uk_amd_no_alloc_scratch_bytes())

    def set_k_slices(self, n: int):
        """K slices across workgroups of the thin mmt4d kernels on this thread
        (0 = choose, 1 = never split)."""
        self.lib.iree_uk_amd_set_k_slices(n)

    def set_streamed_weights(self, on: bool):
        """Hint of this thread: the weights of the decode-shaped mmt4d calls
        that follow come from HBM every time (non-temporal loads)."""
        self.lib.iree_uk_amd_set_streamed_weights(1 if on else 0)

    def last_k_slices(self) -> int:
        return int(self.lib.iree_uk_amd_last_k_slices())

    def mmt4d_info(self, M0, N0, K0, flags, cpu_data=None) -> int:
        return int(self.lib.iree_uk_mmt4d_info(M0, N0, K0, flags, cpu_data))

    def pack(self, inp, in_offset, in_stride0, in_stride1, out, out_offset,
             out_stride0, out_stride1, in_size0, in_size1, out_size0, out_size1,
             out_size2, out_size3, padding_value, flags, cpu_data=None):
        self.lib.iree_uk_pack(inp, in_offset, in_stride0, in_stride1, out,
                              out_offset, out_stride0, out_stride1, in_size0,
                              in_size1, out_size0, out_size1, out_size2,
                              out_size3, padding_value, flags, cpu_data)
        self._check()

    def unpack(self, inp, in_offset, in_stride0, in_stride1, out, out_offset,
               out_stride0, out_stride1, in_size0, in_size1, in_size2, in_size3,
               out_size0, out_size1, flags, cpu_data=None):
        self.lib.iree_uk_unpack(inp, in_offset, in_stride0, in_stride1, out,
                                out_offset, out_stride0, out_stride1, in_size0,
                                in_size1, in_size2, in_size3, out_size0,
                                out_size1, flags, cpu_data)
        self._check()

    def mmt4d_unpack(self, lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0,
                     out, out_offset, out_stride0, out_size0, out_size1, M, N, K,
                     M0, N0, K0, flags, cpu_data=None):
        """mmt4d straight into a row-major out_size0 x out_size1 matrix."""
        self.lib.iree_uk_amd_mmt4d_unpack(lhs, lhs_offset, lhs_stride0, rhs, rhs_offset,
                                          rhs_stride0, out, out_offset, out_stride0,
                                          out_size0, out_size1, M, N, K, M0, N0, K0,
                                          flags, cpu_data)
        self._check()

    def mmt4d_dequant_unpack(self, lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0,
                             acc, acc_offset, acc_stride0, out, out_offset, out_stride0,
                             out_size0, out_size1, row_scale, col_scale, M, N, K,
                             M0, N0, K0, flags, cpu_data=None):
        """mmt4d into a row-major f32 matrix, scaled per row and per column;
        `acc` is the tiled accumulator input read with ACCUMULATE."""
        self.lib.iree_uk_amd_mmt4d_dequant_unpack(
            lhs, lhs_offset, lhs_stride0, rhs, rhs_offset, rhs_stride0, acc, acc_offset,
            acc_stride0, out, out_offset, out_stride0, out_size0, out_size1, row_scale,
            col_scale, M, N, K, M0, N0, K0, flags, cpu_data)
        self._check()

    def conv_nchwc(self, inp, input_offset, input_stride_n, input_stride_ic_outer,
                   input_stride_h, flt, filter_offset, filter_stride_oc_outer,
                   filter_stride_ic_outer, filter_stride_fh, out, output_offset,
                   output_stride_n, output_stride_oc_outer, output_stride_oh, N, OC_outer, OH,
                   OW, IC_outer, FH, FW, k0, c0, stride_h, stride_w, flags, cpu_data=None):
        self.lib.iree_uk_conv_nchwc(inp, input_offset, input_stride_n, input_stride_ic_outer,
                                    input_stride_h, flt, filter_offset, filter_stride_oc_outer,
                                    filter_stride_ic_outer, filter_stride_fh, out, output_offset,
                                    output_stride_n, output_stride_oc_outer, output_stride_oh, N,
                                    OC_outer, OH, OW, IC_outer, FH, FW, k0, c0, stride_h,
                                    stride_w, flags, cpu_data)
        self._check()

    # ---------------------------------------------------------------- probes
    def probe_mfma_peak(self, type_flags, operands, operand_bytes, iters, sink, stream,
                        workgroups=0) -> float:
        """Operations per second of an MFMA-only loop (see the header)."""
        rate = ctypes.c_double(0.0)
        st = self.lib.iree_uk_amd_probe_mfma_peak(type_flags, operands, operand_bytes, iters,
                                                  workgroups, sink, stream, ctypes.byref(rate))
        if st != 0:
            raise RuntimeError(f"iree_uk_amd_probe_mfma_peak: status {st}")
        return rate.value

    def probe_copy2d(self, src, src_pitch, dst, dst_pitch, row_bytes, rows, iters, stream) -> float:
        """Average seconds per plain 2-D copy between two pitches."""
        sec = ctypes.c_double(0.0)
        st = self.lib.iree_uk_amd_probe_copy2d(src, src_pitch, dst, dst_pitch, row_bytes, rows,
                                               iters, stream, ctypes.byref(sec))
        if st != 0:
            raise RuntimeError(f"iree_uk_amd_probe_copy2d: status {st}")
        return sec.value

    def probe_mfma_peak_waves(self, operands, operand_bytes, iters, waves_per_simd, sink, stream) -> float:
        """Operations per second of the s8 MFMA-only loop with 1 or 2 waves on
        every SIMD."""
        rate = ctypes.c_double(0.0)
        st = self.lib.iree_uk_amd_probe_mfma_peak_waves(operands, operand_bytes, iters, waves_per_simd,
                                                        sink, stream, ctypes.byref(rate))
        if st != 0:
            raise RuntimeError(f"iree_uk_amd_probe_mfma_peak_waves: status {st}")
        return rate.value

    def probe_copy2d_variants(self, src, src_pitch, dst, dst_pitch, row_bytes, rows, iters, stream):
        """(seconds of the fastest copy variant, [seconds of each of the five
        variants]); the last variant writes whole 128-byte lines only."""
        sec = ctypes.c_double(0.0)
        per = (ctypes.c_double * 5)()
        st = self.lib.iree_uk_amd_probe_copy2d_variants(src, src_pitch, dst, dst_pitch, row_bytes, rows,
                                                        iters, stream, ctypes.byref(sec), per)
        if st != 0:
            raise RuntimeError(f"iree_uk_amd_probe_copy2d_variants: status {st}")
        return sec.value, list(per)

    def probe_ds_read_tr16(self, lane_index_ptr, out_ptr, lds_values, stream) -> None:
        st = self.lib.iree_uk_amd_probe_ds_read_tr16(lane_index_ptr, out_ptr, lds_values, stream)
        if st != 0:
            raise RuntimeError(f"iree_uk_amd_probe_ds_read_tr16: status {st}")

    # --------------------------------------------------------------- control
    def _check(self):
        if self._violations:
            msg = "; ".join(self._violations)
            self._violations.clear()
            raise ContractViolation(msg)
        st = self.lib.iree_uk_amd_last_status()
        if st not in (0,):
            raise RuntimeError(
                f"iree_uk_amd: status {st}: "
                f"{self.lib.iree_uk_amd_last_status_string().decode()}")

    def raise_on_violation(self, enable: bool = True):
        """Routes contract violations to ContractViolation instead of the
        default print-and-abort handler."""
        if not enable:
            self.lib.iree_uk_amd_set_assert_handler(None)
            self._handler_ref = None
            return

        def handler(file, line, function, condition):
            self._violations.append(
                f"{function.decode()}: assertion failed: {condition.decode()}")

        self._handler_ref = ASSERT_HANDLER(handler)
        self.lib.iree_uk_amd_set_assert_handler(
            ctypes.cast(self._handler_ref, _vp))

    def set_stream(self, hip_stream: int | None):
        self.lib.iree_uk_amd_set_stream(hip_stream)

    def synchronize(self):
        st = self.lib.iree_uk_amd_synchronize()
        if st:
            raise RuntimeError(f"iree_uk_amd_synchronize: status {st}")

    def set_pointer_mode(self, mode: int):
        self.lib.iree_uk_amd_set_pointer_mode(mode)

    def set_kernel_mode(self, mode: int):
        self.lib.iree_uk_amd_set_kernel_mode(mode)

    def mfma_decline_count(self) -> int:
        """Calls of this thread that the info query advertises an MFMA kernel
        for but that the scalar kernel served."""
        return int(self.lib.iree_uk_amd_mfma_decline_count())

    def set_persistent_workgroups(self, n: int):
        """Workgroups the persistent mmt4d kernels launch on this thread
        (0 = one per compute unit)."""
        self.lib.iree_uk_amd_set_persistent_workgroups(n)

    def last_kernel_name(self) -> str:
        return self.lib.iree_uk_amd_last_kernel_name().decode()

    def timing_begin(self):
        """Starts per-kernel device timing of this thread's calls."""
        self.lib.iree_uk_amd_timing_begin()

    def timing_end(self, capacity: int = 4096):
        """Returns [(kind, microseconds)] for every kernel launched since
        timing_begin, in launch order; kind is 0 pack, 1 unpack, 2 mmt4d."""
        us = (ctypes.c_double * capacity)()
        kinds = (ctypes.c_int * capacity)()
        n = self.lib.iree_uk_amd_timing_end(us, kinds, capacity)
        n = min(n, capacity)
        return [(kinds[i], us[i]) for i in range(n)]

    def staging_bytes(self) -> int:
        """Device bytes the calling thread's host-operand staging arena holds."""
        return int(self.lib.iree_uk_amd_staging_bytes())

    def device_alloc_count(self) -> int:
        """hipMalloc calls the library has made in this process so far."""
        return int(self.lib.iree_uk_amd_device_alloc_count())

    def workspace_bytes(self) -> int:
        """Bytes of K-split workspaces and prepared-operand buffers the calling thread holds."""
        return int(self.lib.iree_uk_amd_workspace_bytes())

    def release_workspaces(self) -> int:
        """Frees them; 0 or a hipError_t value."""
        return int(self.lib.iree_uk_amd_release_workspaces())

    def release_staging(self) -> int:
        """Frees the calling thread's staging arena; 0 or a hipError_t value."""
        return int(self.lib.iree_uk_amd_release_staging())

    def device_count(self) -> int:
        return int(self.lib.iree_uk_amd_device_count())

    def version(self) -> str:
        return self.lib.iree_uk_amd_version().decode()


_lib: UKernelLibrary | None = None


def load() -> UKernelLibrary:
    """Loads the library once per process; raises ImportError if it is not built."""
    global _lib
    if _lib is None:
        _lib = UKernelLibrary()
    return _lib
