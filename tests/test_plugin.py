"""The library as a HAL executable plugin: query / load / resolve follow the
contract of runtime/src/iree/hal/local/executable_plugin.h:175-191,404-461, and
the resolved import thunks take the packed parameter structs that compiled
LLVMCPU code passes (compiler/src/iree/compiler/Codegen/LLVMCPU/DispatchABI.cpp:
1170-1186: results, then arguments, then extra fields)."""
import ctypes

import numpy as np
import pytest

from iree_amd import ukernel as uk

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64


class Header(ctypes.Structure):  # executable_plugin.h:152-173
    _fields_ = [("version", ctypes.c_uint32), ("name", ctypes.c_char_p),
                ("description", ctypes.c_char_p), ("features", ctypes.c_uint32),
                ("sanitizer", ctypes.c_int32), ("reserved", ctypes.c_uint64 * 8)]


class ResolveParams(ctypes.Structure):  # executable_plugin.h:389-394
    _fields_ = [("count", ctypes.c_size_t), ("symbol_names", ctypes.POINTER(ctypes.c_char_p)),
                ("out_fn_ptrs", ctypes.POINTER(_vp)), ("out_fn_contexts", ctypes.POINTER(_vp))]


LOAD_FN = ctypes.CFUNCTYPE(_vp, _vp, ctypes.c_size_t, _vp, ctypes.POINTER(_vp))
UNLOAD_FN = ctypes.CFUNCTYPE(None, _vp)
RESOLVE_FN = ctypes.CFUNCTYPE(_vp, _vp, ctypes.POINTER(ResolveParams),
                              ctypes.POINTER(ctypes.c_uint32))
IMPORT_FN = ctypes.CFUNCTYPE(ctypes.c_int, _vp, _vp, _vp)  # executable_library.h:157-158


class PluginV0(ctypes.Structure):  # executable_plugin.h:404-461
    _fields_ = [("header", ctypes.POINTER(Header)), ("load", LOAD_FN), ("unload", UNLOAD_FN),
                ("resolve", RESOLVE_FN)]


class Mmt4dImport(ctypes.Structure):  # i32 result, then mmt4d_internal.h:14-32
    _fields_ = [("unused_result", ctypes.c_int32),
                ("lhs_buffer", _vp), ("lhs_offset", _i64), ("lhs_stride0", _i64),
                ("rhs_buffer", _vp), ("rhs_offset", _i64), ("rhs_stride0", _i64),
                ("out_buffer", _vp), ("out_offset", _i64), ("out_stride0", _i64),
                ("M", _i64), ("N", _i64), ("K", _i64),
                ("M0", ctypes.c_int32), ("N0", ctypes.c_int32), ("K0", ctypes.c_int32),
                ("flags", ctypes.c_uint32), ("cpu_data", _vp)]


class PackImport(ctypes.Structure):  # i32 result, then pack_internal.h:12-30
    _fields_ = [("unused_result", ctypes.c_int32),
                ("in_buffer", _vp), ("in_offset", _i64), ("in_stride0", _i64), ("in_stride1", _i64),
                ("out_buffer", _vp), ("out_offset", _i64), ("out_stride0", _i64),
                ("out_stride1", _i64), ("in_size0", _i64), ("in_size1", _i64),
                ("out_size0", _i64), ("out_size1", _i64), ("out_size2", _i64),
                ("out_size3", _i64), ("padding_value", ctypes.c_uint64),
                ("flags", ctypes.c_uint32), ("cpu_data", _vp)]


class UnpackImport(ctypes.Structure):  # i32 result, then unpack_internal.h:12-29
    _fields_ = [("unused_result", ctypes.c_int32),
                ("in_buffer", _vp), ("in_offset", _i64), ("in_stride0", _i64), ("in_stride1", _i64),
                ("out_buffer", _vp), ("out_offset", _i64), ("out_stride0", _i64),
                ("out_stride1", _i64), ("in_size0", _i64), ("in_size1", _i64),
                ("in_size2", _i64), ("in_size3", _i64), ("out_size0", _i64),
                ("out_size1", _i64), ("flags", ctypes.c_uint32), ("cpu_data", _vp)]


def _query(lib, max_version):
    fn = lib.lib.iree_hal_executable_plugin_query
    fn.restype = ctypes.POINTER(PluginV0)
    fn.argtypes = [ctypes.c_uint32, _vp]
    return fn(max_version, None)


def _resolve(plugin, names, preset=None):
    n = len(names)
    c_names = (ctypes.c_char_p * n)(*[s.encode() for s in names])
    ptrs = (_vp * n)(*(preset or [None] * n))
    ctxs = (_vp * n)()
    params = ResolveParams(n, c_names, ptrs, ctxs)
    resolution = ctypes.c_uint32(0xFFFF)
    self_ptr = _vp(0x1234)
    assert plugin.load(None, 0, None, ctypes.byref(self_ptr)) in (None, 0)
    status = plugin.resolve(self_ptr, ctypes.byref(params), ctypes.byref(resolution))
    plugin.unload(self_ptr)
    return (status or 0), resolution.value, [p for p in ptrs]


def test_query_versions_and_header(lib):
    assert not _query(lib, 0)                      # caller too old: NULL
    p = _query(lib, 1)
    assert p and p.contents.header.contents.version == 1
    assert p.contents.header.contents.name == b"iree_uk_amd"
    assert p.contents.header.contents.features == 0   # not STANDALONE: needs the HIP runtime
    assert p.contents.header.contents.sanitizer == 0
    assert _query(lib, 7)                          # a newer caller may load 0.1


def test_resolve_required_optional_and_preset(lib):
    plugin = _query(lib, 1).contents
    st, res, ptrs = _resolve(plugin, ["iree_uk_conv_nchwc", "iree_uk_mmt4d", "iree_uk_pack",
                                      "iree_uk_unpack"])
    assert st == 0 and res == 0 and all(ptrs) and len(set(ptrs)) == 4
    # optional and unknown: OK with the MISSING_OPTIONAL bit, entry left NULL
    st, res, ptrs = _resolve(plugin, ["?iree_uk_conv", "?iree_uk_mmt4d"])
    assert st == 0 and res == 1 and ptrs[0] is None and ptrs[1]
    # required and unknown: NOT_FOUND (5), what is available still filled in
    st, res, ptrs = _resolve(plugin, ["iree_uk_conv", "iree_uk_pack"])
    assert st == 5 and ptrs[0] is None and ptrs[1]
    # entries another provider already resolved are left alone
    st, res, ptrs = _resolve(plugin, ["iree_uk_mmt4d"], preset=[0xABCD0])
    assert st == 0 and ptrs[0] == 0xABCD0


def test_import_struct_layouts_match_the_params_structs():
    # one i32 result, then the params struct at its natural (8-byte) alignment
    assert Mmt4dImport.lhs_buffer.offset == 8 and ctypes.sizeof(Mmt4dImport) == 8 + 120
    assert PackImport.in_buffer.offset == 8 and PackImport.cpu_data.offset == 8 + 128
    assert UnpackImport.in_buffer.offset == 8 and UnpackImport.cpu_data.offset == 8 + 120


@pytest.mark.gpu
def test_import_thunks_compute_on_host_buffers(gpu, oracle):
    """What a compiled CPU dispatch does: host pointers in, result in host
    memory when the import returns 0."""
    lib, torch = gpu
    lib.set_kernel_mode(uk.KERNEL_MODE_AUTO)
    lib.set_pointer_mode(uk.POINTER_MODE_AUTO)
    plugin = _query(lib, 1).contents
    st, _, ptrs = _resolve(plugin, ["iree_uk_mmt4d", "iree_uk_pack", "iree_uk_unpack"])
    assert st == 0
    mmt4d, pack, unpack = (IMPORT_FN(p) for p in ptrs)
    rng = np.random.default_rng(5)
    M, N, K, M0, N0, K0 = 70, 50, 96, 16, 16, 16
    M1, N1, K1 = -(-M // M0), -(-N // N0), K // K0
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    bt = rng.integers(-128, 128, (N, K), dtype=np.int8)
    lhs4 = np.zeros(M1 * K1 * M0 * K0, np.int8)
    rhs4 = np.zeros(N1 * K1 * N0 * K0, np.int8)
    for src, rows, dst, o0, t0 in ((a, M, lhs4, M1, M0), (bt, N, rhs4, N1, N0)):
        p = PackImport(0, src.ctypes.data, 0, K, 1, dst.ctypes.data, 0, K1 * t0 * K0, t0 * K0,
                       rows, K, o0, K1, t0, K0, 0, uk.PACK_TYPE_I8I8, None)
        assert pack(ctypes.addressof(p), None, None) == 0
    want_l, want_r = np.zeros_like(lhs4), np.zeros_like(rhs4)
    oracle.pack(a.reshape(-1), 0, K, 1, want_l, 0, K1 * M0 * K0, M0 * K0, M, K, M1, K1, M0, K0, 0,
                uk.PACK_TYPE_I8I8)
    oracle.pack(bt.reshape(-1), 0, K, 1, want_r, 0, K1 * N0 * K0, N0 * K0, N, K, N1, K1, N0, K0, 0,
                uk.PACK_TYPE_I8I8)
    assert np.array_equal(lhs4, want_l) and np.array_equal(rhs4, want_r)
    out4 = rng.integers(-1000, 1000, M1 * N1 * M0 * N0).astype(np.int32)
    want4 = out4.copy()
    flags = uk.MMT4D_TYPE_S8S8S32 | uk.MMT4D_ACCUMULATE | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    p = Mmt4dImport(0, lhs4.ctypes.data, 0, K1 * M0 * K0, rhs4.ctypes.data, 0, K1 * N0 * K0,
                    out4.ctypes.data, 0, N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags, None)
    assert mmt4d(ctypes.addressof(p), None, None) == 0
    oracle.mmt4d(lhs4, 0, K1 * M0 * K0, rhs4, 0, K1 * N0 * K0, want4, 0, N1 * M0 * N0,
                 M1, N1, K1, M0, N0, K0, flags)
    assert np.array_equal(out4, want4)
    out = np.full(M * N, -7, np.int32)
    want = out.copy()
    p = UnpackImport(0, out4.ctypes.data, 0, N1 * M0 * N0, M0 * N0, out.ctypes.data, 0, N, 1,
                     M1, N1, M0, N0, M, N, uk.UNPACK_TYPE_I32I32, None)
    assert unpack(ctypes.addressof(p), None, None) == 0
    oracle.unpack(want4, 0, N1 * M0 * N0, M0 * N0, want, 0, N, 1, M1, N1, M0, N0, M, N,
                  uk.UNPACK_TYPE_I32I32)
    assert np.array_equal(out, want)
