"""The C-ABI library loads, exports every symbol that include/iree_uk_amd.h
declares, and its host layer validates like the reference. No kernel is
launched: runs without a GPU."""
import ctypes
import os
import re

import numpy as np
import pytest

from iree_amd import ukernel as uk

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "iree_uk_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(iree_uk_\w+)\s*\(", text))
    names -= {"iree_uk_amd_assert_handler_t"}
    return sorted(names)


def test_exports_every_declared_symbol(lib):
    names = _declared_functions()
    assert len(names) >= 18, names
    for n in names:
        assert hasattr(lib.lib, n), f"{n} is declared in the header but not exported"


def test_struct_layouts_match_reference_field_order():
    # iree_uk_mmt4d_params_t is 120 bytes on LP64 (9 pointer/index fields of 8,
    # 3 index sizes of 8, 3 int32 + flags, then the cpu_data pointer).
    class P(ctypes.Structure):
        _fields_ = [("lhs_buffer", ctypes.c_void_p), ("lhs_offset", ctypes.c_int64),
                    ("lhs_stride0", ctypes.c_int64), ("rhs_buffer", ctypes.c_void_p),
                    ("rhs_offset", ctypes.c_int64), ("rhs_stride0", ctypes.c_int64),
                    ("out_buffer", ctypes.c_void_p), ("out_offset", ctypes.c_int64),
                    ("out_stride0", ctypes.c_int64), ("M", ctypes.c_int64),
                    ("N", ctypes.c_int64), ("K", ctypes.c_int64), ("M0", ctypes.c_int32),
                    ("N0", ctypes.c_int32), ("K0", ctypes.c_int32),
                    ("flags", ctypes.c_uint32), ("cpu_data", ctypes.c_void_p)]
    assert ctypes.sizeof(P) == 120


def test_mmt4d_p_early_return_through_struct(lib):
    class P(ctypes.Structure):
        _fields_ = [("lhs_buffer", ctypes.c_void_p), ("lhs_offset", ctypes.c_int64),
                    ("lhs_stride0", ctypes.c_int64), ("rhs_buffer", ctypes.c_void_p),
                    ("rhs_offset", ctypes.c_int64), ("rhs_stride0", ctypes.c_int64),
                    ("out_buffer", ctypes.c_void_p), ("out_offset", ctypes.c_int64),
                    ("out_stride0", ctypes.c_int64), ("M", ctypes.c_int64),
                    ("N", ctypes.c_int64), ("K", ctypes.c_int64), ("M0", ctypes.c_int32),
                    ("N0", ctypes.c_int32), ("K0", ctypes.c_int32),
                    ("flags", ctypes.c_uint32), ("cpu_data", ctypes.c_void_p)]
    p = P(M=0, N=3, K=3, M0=2, N0=2, K0=2, flags=0x202)
    lib.lib.iree_uk_mmt4d_p(ctypes.byref(p))
    assert lib.lib.iree_uk_amd_last_status() == 0


def test_flag_values_match_exported_bits():
    # runtime/src/iree/builtins/ukernel/exported_bits.h and the lit checks of
    # compiler/src/iree/compiler/Codegen/Common/CPU/test/lower_to_ukernel_ops.mlir
    # (:240 f16f16f16 with all three bit flags = 1796; :303 pack i8 = 2;
    # :331 f16 = 4; :360 bf16 = 5).
    assert (uk.MMT4D_TYPE_F16F16F16 | uk.MMT4D_ACCUMULATE |
            uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION |
            uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == 1796
    assert uk.PACK_TYPE_I8I8 == 2 and uk.PACK_TYPE_F16F16 == 4 and uk.PACK_TYPE_BF16BF16 == 5
    assert uk.MMT4D_TYPE_S8S8S32 == 2 and uk.MMT4D_TYPE_S8S4S32 == 0x0A
    text = open(os.path.join(ROOT, "include", "iree_uk_amd.h")).read()
    for name, val in (("IREE_UK_FLAG_MMT4D_TYPE_END", 0x0B),
                      ("IREE_UK_FLAG_MMT4D_ACCUMULATE", 0x100),
                      ("IREE_UK_FLAG_PACK_TRANSPOSE_OUTER", 0x200),
                      ("IREE_UK_FLAG_UNPACK_TYPE_I32I32", 0x03)):
        m = re.search(name + r"\s*=\s*(0x[0-9A-Fa-f]+)", text)
        assert m and int(m.group(1), 16) == val, name


def test_early_returns_need_no_device(lib):
    # mmt4d.c:106-114, pack.c:106-109, unpack.c:84-86: nothing is touched, so
    # null buffers are fine and no HIP call is made.
    lib.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 0, 5, 7, 3, 4, 2, 0x202)
    lib.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 5, 0, 7, 3, 4, 2, 0x202)
    lib.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 5, 7, 0, 3, 4, 2, 0x302)
    lib.pack(None, 0, 0, 1, None, 0, 0, 6, 0, 0, 0, 1, 2, 3, 0, uk.PACK_TYPE_I8I8)
    lib.pack(None, 0, 0, 1, None, 0, 0, 0, 0, 0, 1, 1, 0, 3, 0, uk.PACK_TYPE_I8I8)
    lib.unpack(None, 0, 0, 6, None, 0, 0, 1, 1, 1, 2, 3, 0, 3, uk.UNPACK_TYPE_F32F32)
    assert lib.last_kernel_name() == ""


@pytest.mark.parametrize("call,needle", [
    (lambda L: L.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 1, 1, 1, 2, 2, 2, 0x0B | 0x200), "mmt4d_type_bits"),
    (lambda L: L.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 1, 1, 1, 2, 2, 2, 0x802), "allflags"),
    (lambda L: L.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, -1, 1, 1, 2, 2, 2, 0x202), "p->M"),
    (lambda L: L.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 1, 1, 1, 2, 2, 1 << 15, 0x202), "p->K0"),
    (lambda L: L.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 1, 1, 1, 2, 2, 3, 0x20A), "rhs_bits"),
    (lambda L: L.mmt4d(None, 0, 0, None, 0, 0, None, 0, 0, 1, 1, 1, 7, 3, 5, 0x002), "fallback not enabled"),
    (lambda L: L.pack(None, 0, 5, 1, None, 0, 12, 5, 3, 5, 2, 2, 2, 3, 0, 0x002), "out_stride1"),
    (lambda L: L.pack(None, 0, 5, 1, None, 0, 12, 6, 3, 5, 1, 2, 2, 3, 0, 0x002), "in_size0"),
    (lambda L: L.pack(None, 0, 5, 1, None, 0, 12, 6, 3, 5, 2, 2, 2, 3, 0, 0x006), "es != 0"),
    (lambda L: L.pack(None, 0, 5, 1, None, 0, 12, 6, 3, 5, 2, 2, 2, 3, 0, 0x402), "allflags"),
    (lambda L: L.pack(None, 0, 4096, 1, None, 0, 8192, 8192, 64, 128, 1, 1, 64, 128, 0, 0x002), "4096"),
    (lambda L: L.unpack(None, 0, 12, 6, None, 0, 5, 1, 2, 2, 2, 3, 3, 5, 0x002), "es != 0"),
    (lambda L: L.unpack(None, 0, 12, 5, None, 0, 5, 1, 2, 2, 2, 3, 3, 5, 0x003), "in_stride1"),
    (lambda L: L.unpack(None, 0, 12, 6, None, 0, 5, 1, 2, 2, 2, 3, 5, 5, 0x003), "out_size0"),
])
def test_contract_violations_reach_the_hook(lib, call, needle):
    """Same conditions as the reference's validate functions
    (mmt4d.c:12-48, pack.c:51-104, unpack.c:31-81)."""
    with pytest.raises(uk.ContractViolation) as e:
        call(lib)
    assert needle in str(e.value)
    assert lib.lib.iree_uk_amd_last_status() == -1


def test_mmt4d_info_reports_mfma_shapes(lib):
    # No MFMA kernel for odd tiles; the generic flag does not matter for info.
    assert lib.mmt4d_info(7, 3, 5, uk.MMT4D_TYPE_S8S8S32) == 0
    for flags, tile in ((uk.MMT4D_TYPE_S8S8S32, (16, 16, 2)),
                        (uk.MMT4D_TYPE_S8S8S32, (32, 16, 8)),
                        (uk.MMT4D_TYPE_F16F16F32, (16, 16, 16)),
                        (uk.MMT4D_TYPE_BF16BF16F32, (16, 16, 2)),
                        (uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32, (16, 16, 32))):
        assert lib.mmt4d_info(*tile, flags) == 1, (hex(flags), tile)


def test_query_tile_sizes(lib):
    class P(ctypes.Structure):
        _fields_ = [("flags", ctypes.c_uint32), ("size0", ctypes.c_int64),
                    ("size1", ctypes.c_int64), ("cpu_data", ctypes.c_void_p)]

    class O(ctypes.Structure):
        _fields_ = [("tile_size0", ctypes.c_int64), ("tile_size1", ctypes.c_int64)]

    def q(op, role):
        p, o = P(flags=op | role, size0=1024, size1=1024), O()
        lib.lib.iree_uk_query_tile_sizes_2d(ctypes.byref(p), ctypes.byref(o))
        return o.tile_size0, o.tile_size1

    m, k = q(0x0200, 1)
    n, k2 = q(0x0200, 2)
    m2, n2 = q(0x0200, 3)
    assert (m, n, k) == (m2, n2, k2)
    # The tiles the query hands out are ones the MFMA kernels serve.
    assert lib.mmt4d_info(m, n, k, uk.MMT4D_TYPE_S8S8S32) == 1
    m, k = q(0x0300, 1)
    n, _ = q(0x0300, 2)
    assert lib.mmt4d_info(m, n, k, uk.MMT4D_TYPE_F16F16F32) == 1


def test_product_does_not_reference_the_oracle():
    """The shipped package must not import, load or name anything in oracle/."""
    pkg = os.path.join(ROOT, "iree_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".c", ".h", ".hip")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
