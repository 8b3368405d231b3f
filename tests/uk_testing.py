"""Shared helpers for the ukernel tests: seeded input generators and the case
lists that mirror the reference's own unit tests
(runtime/src/iree/builtins/ukernel/tools/{pack,unpack,mmt4d}_test.c)."""
from __future__ import annotations

import dataclasses
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from iree_amd import ukernel as uk  # noqa: E402


class Lcg:
    """minstd-like generator of the reference tests (tools/util.c:73-103). The
    multiply wraps in 32 bits before the modulo, as in the C code."""

    def __init__(self, seed: int = 1):
        self.state = seed & 0xFFFFFFFF

    def u32(self) -> int:
        self.state = ((self.state * 48271) & 0xFFFFFFFF) % 2147483647
        return self.state

    def u64(self) -> int:
        hi = self.u32()
        return (hi << 32) + self.u32()

    def r16(self) -> int:
        return (self.u32() >> 8) & 0xFFFF

    def bit(self) -> int:
        return self.r16() & 1


# --------------------------------------------------------------------------
# element types
# --------------------------------------------------------------------------

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 bit patterns (finite inputs)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f8e4m3fn_table() -> np.ndarray:
    """All 256 decodings from the closed form: (-1)^s * 2^(e-7) * (1+m/8), or
    m * 2^-9 when e == 0; S.1111.111 is NaN."""
    t = np.zeros(256, dtype=np.float32)
    for v in range(256):
        s = -1.0 if v & 0x80 else 1.0
        e = (v >> 3) & 0xF
        m = v & 7
        if e == 0xF and m == 7:
            t[v] = np.nan
        elif e == 0:
            t[v] = s * m * 2.0 ** -9
        else:
            t[v] = s * (1 + m / 8.0) * 2.0 ** (e - 7)
    return t


def f32_to_f8e4m3fn_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even cast of finite f32 values with |x| <= 448 to
    E4M3FN, by nearest-value search over the 127 non-negative finite codes
    (ties to the even code)."""
    table = f8e4m3fn_table()[:0x7F].astype(np.float64)  # 0 .. 448, increasing
    a = np.abs(np.asarray(x, dtype=np.float64)).ravel()
    hi = np.searchsorted(table, a, side="left").clip(0, 0x7E)
    lo = (hi - 1).clip(0, 0x7E)
    dlo = np.abs(a - table[lo])
    dhi = np.abs(table[hi] - a)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code |= (np.signbit(np.asarray(x, dtype=np.float64)).ravel().astype(np.uint8) << 7)
    return code.reshape(np.shape(x))


def random_elements(rng: np.random.Generator, kind: str, n: int) -> np.ndarray:
    """Buffers in the style of tools/util.c:131-165: small integer values so
    that float products and sums are exact whatever the summation order; full
    range for 8-bit integers. Returns the storage dtype (uint16 for f16/bf16
    bit patterns, uint8 for f8 and packed 4-bit)."""
    if kind == "f32":
        return rng.integers(-2, 2, n).astype(np.float32)
    if kind == "f16":
        return rng.integers(-8, 8, n).astype(np.float16).view(np.uint16)
    if kind == "bf16":
        return f32_to_bf16_bits(rng.integers(-2, 2, n).astype(np.float32))
    if kind == "f8":
        return f32_to_f8e4m3fn_bits(rng.integers(-4, 5, n).astype(np.float32))
    if kind == "s8":
        return rng.integers(-128, 128, n).astype(np.int8)
    if kind in ("u4x2", "s4x2"):
        return rng.integers(0, 256, n).astype(np.uint8)
    if kind == "s16":
        return rng.integers(-512, 1536, n).astype(np.int16)
    if kind == "s32":
        return rng.integers(-512, 1536, n).astype(np.int32)
    raise ValueError(kind)


# (lhs kind, rhs kind, out kind) per mmt4d type value.
MMT4D_KINDS = {
    uk.MMT4D_TYPE_F32F32F32: ("f32", "f32", "f32"),
    uk.MMT4D_TYPE_S8S8S32: ("s8", "s8", "s32"),
    uk.MMT4D_TYPE_F16F16F32: ("f16", "f16", "f32"),
    uk.MMT4D_TYPE_F16F16F16: ("f16", "f16", "f16"),
    uk.MMT4D_TYPE_BF16BF16F32: ("bf16", "bf16", "f32"),
    uk.MMT4D_TYPE_BF16BF16BF16: ("bf16", "bf16", "bf16"),
    uk.MMT4D_TYPE_S16S16S32: ("s16", "s16", "s32"),
    uk.MMT4D_TYPE_S16U4S32: ("s16", "u4x2", "s32"),
    uk.MMT4D_TYPE_S16S8S32: ("s16", "s8", "s32"),
    uk.MMT4D_TYPE_S8S4S32: ("s8", "s4x2", "s32"),
    uk.MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: ("f8", "f8", "f32"),
}

KIND_BITS = {"f32": 32, "f16": 16, "bf16": 16, "f8": 8, "s8": 8, "u4x2": 4,
             "s4x2": 4, "s16": 16, "s32": 32}

PACK_KINDS = {uk.PACK_TYPE_F32F32: "f32", uk.PACK_TYPE_I8I8: "s8",
              uk.PACK_TYPE_I32I32: "s32", uk.PACK_TYPE_F16F16: "f16",
              uk.PACK_TYPE_BF16BF16: "bf16"}


# --------------------------------------------------------------------------
# cases
# --------------------------------------------------------------------------

@dataclasses.dataclass
class PackCase:
    flags: int
    in_size0: int
    in_size1: int
    out_size0: int
    out_size1: int
    out_size2: int
    out_size3: int
    in_stride0: int
    in_stride1: int
    out_stride0: int
    in_offset: int
    out_offset: int
    padding_value: int

    @property
    def elem_bytes(self):
        return uk.PACK_TYPE_BYTES[self.flags & 0xFF]

    @property
    def out_stride1(self):
        return self.out_size2 * self.out_size3

    def label(self):
        return (f"flags={self.flags:#x} in={self.in_size0}x{self.in_size1} "
                f"out={self.out_size0}x{self.out_size1}x{self.out_size2}x{self.out_size3} "
                f"is=({self.in_stride0},{self.in_stride1}) os0={self.out_stride0} "
                f"off=({self.in_offset},{self.out_offset})")


def pack_cases(type_flag: int, tile0: int, tile1: int, seed: int,
               outer_shapes=((0, 1), (1, 0), (1, 1), (3, 2), (9, 33)),
               max_offset: int = 65535):
    """The case grid of tools/pack_test.c:127-196: outer shapes x transposes x
    {no padding, one incomplete tile, 16 extra all-padding tiles}, random
    strides (tight or not), random offsets and a random 64-bit padding value."""
    g = Lcg(seed)
    for (s0, s1) in outer_shapes:
        for ti in (0, 1):
            for to in (0, 1):
                for pad in ("none", "one_incomplete_tile", "a_lot"):
                    o0, o1 = s0, s1
                    if pad == "a_lot":
                        o0 += 16
                        o1 += 16
                    flags = type_flag
                    out_size0, out_size1 = o0, o1
                    if to:
                        flags |= uk.PACK_TRANSPOSE_OUTER
                        out_size0, out_size1 = out_size1, out_size0
                    t0, t1 = tile0, tile1
                    if ti:
                        flags |= uk.PACK_TRANSPOSE_INNER
                        t0, t1 = t1, t0
                    in0, in1 = o0 * t0, o1 * t1
                    if pad == "one_incomplete_tile":
                        in0 = max(0, in0 - g.r16() % t0)
                        in1 = max(0, in1 - g.r16() % t1)
                    if pad == "a_lot":
                        in0 = s0 * t0
                        in1 = s1 * t1
                    padding = g.u64()
                    in_stride1 = 1 + g.bit()
                    in_stride0 = in1 * in_stride1 + g.bit()
                    out_stride0 = out_size1 * tile0 * tile1 + g.bit()
                    yield PackCase(flags, in0, in1, out_size0, out_size1, tile0,
                                   tile1, in_stride0, in_stride1, out_stride0,
                                   g.r16() % (max_offset + 1),
                                   g.r16() % (max_offset + 1), padding)


@dataclasses.dataclass
class UnpackCase:
    flags: int
    in_size0: int
    in_size1: int
    in_size2: int
    in_size3: int
    out_size0: int
    out_size1: int
    in_stride0: int
    out_stride0: int
    out_stride1: int
    in_offset: int
    out_offset: int

    @property
    def elem_bytes(self):
        return uk.PACK_TYPE_BYTES[self.flags & 0xFF]

    @property
    def in_stride1(self):
        return self.in_size2 * self.in_size3

    def label(self):
        return (f"flags={self.flags:#x} in={self.in_size0}x{self.in_size1}x"
                f"{self.in_size2}x{self.in_size3} out={self.out_size0}x{self.out_size1} "
                f"is0={self.in_stride0} os=({self.out_stride0},{self.out_stride1})")


def unpack_cases(type_flag: int, tile0: int, tile1: int, seed: int,
                 outer_shapes=((0, 1), (1, 0), (1, 1), (3, 2), (9, 33)),
                 max_offset: int = 65535):
    """The case grid of tools/unpack_test.c:117-180 (as pack, without the
    all-padding variant being special: outer sizes may exceed the need)."""
    g = Lcg(seed)
    for (s0, s1) in outer_shapes:
        for ti in (0, 1):
            for to in (0, 1):
                for pad in ("none", "one_incomplete_tile", "a_lot"):
                    o0, o1 = s0, s1
                    if pad == "a_lot":
                        o0 += 16
                        o1 += 16
                    flags = type_flag
                    in_size0, in_size1 = o0, o1
                    if to:
                        flags |= uk.UNPACK_TRANSPOSE_OUTER
                        in_size0, in_size1 = in_size1, in_size0
                    t0, t1 = tile0, tile1
                    if ti:
                        flags |= uk.UNPACK_TRANSPOSE_INNER
                        t0, t1 = t1, t0
                    out0, out1 = o0 * t0, o1 * t1
                    if pad == "one_incomplete_tile":
                        out0 = max(0, out0 - g.r16() % t0)
                        out1 = max(0, out1 - g.r16() % t1)
                    if pad == "a_lot":
                        out0 = s0 * t0
                        out1 = s1 * t1
                    out_stride1 = 1 + g.bit()
                    out_stride0 = out1 * out_stride1 + g.bit()
                    in_stride0 = in_size1 * tile0 * tile1 + g.bit()
                    yield UnpackCase(flags, in_size0, in_size1, tile0, tile1,
                                     out0, out1, in_stride0, out_stride0,
                                     out_stride1, g.r16() % (max_offset + 1),
                                     g.r16() % (max_offset + 1))


@dataclasses.dataclass
class Mmt4dCase:
    flags: int
    M: int
    N: int
    K: int
    M0: int
    N0: int
    K0: int
    lhs_stride0: int
    rhs_stride0: int
    out_stride0: int
    lhs_offset: int
    rhs_offset: int
    out_offset: int

    def bits(self):
        return uk.MMT4D_TYPE_BITS[self.flags & 0xFF]

    def label(self):
        return (f"flags={self.flags:#x} MNK={self.M}x{self.N}x{self.K} "
                f"tile={self.M0}x{self.N0}x{self.K0} strides=({self.lhs_stride0},"
                f"{self.rhs_stride0},{self.out_stride0}) off=({self.lhs_offset},"
                f"{self.rhs_offset},{self.out_offset})")


MMT4D_TEST_SHAPES = ((0, 1, 1), (0, 5, 7), (1, 0, 1), (5, 0, 7), (1, 1, 0),
                     (5, 7, 0), (1, 1, 1), (1, 1, 2), (1, 1, 10), (1, 1, 1000),
                     (2, 1, 1), (1, 2, 1), (2, 2, 2), (5, 7, 13))


def _round_up_whole_bytes(v: int, bits: int) -> int:
    while (v * bits) % 8:
        v += 1
    return v


def mmt4d_cases(type_flag: int, M0: int, N0: int, K0: int, seed: int,
                shapes=MMT4D_TEST_SHAPES, extra_flags: int = 0, slack: int = 1):
    """The case grid of tools/mmt4d_test.c:354-404,448-506: shapes x ACCUMULATE
    off/on, strides tight or `slack` elements loose, offsets 0 or `slack`
    (rounded up to whole bytes for 4-bit types). slack=1 is the reference's
    choice; slack=16 keeps operands 16-byte aligned."""
    g = Lcg(seed)
    lb, rb, ob = uk.MMT4D_TYPE_BITS[type_flag]
    for (m, n, k) in shapes:
        if k == 1000 and ob == 16 and (type_flag == uk.MMT4D_TYPE_BF16BF16BF16):
            k = 100  # tools/mmt4d_test.c:456-458
        for acc in (0, 1):
            flags = type_flag | extra_flags | (uk.MMT4D_ACCUMULATE if acc else 0)
            ls = _round_up_whole_bytes(k * M0 * K0 + slack * g.bit(), lb)
            rs = _round_up_whole_bytes(k * N0 * K0 + slack * g.bit(), rb)
            os_ = _round_up_whole_bytes(n * M0 * N0 + slack * g.bit(), ob)
            lo = _round_up_whole_bytes(slack * g.bit(), lb)
            ro = _round_up_whole_bytes(slack * g.bit(), rb)
            oo = _round_up_whole_bytes(slack * g.bit(), ob)
            yield Mmt4dCase(flags, m, n, k, M0, N0, K0, ls, rs, os_, lo, ro, oo)


# --------------------------------------------------------------------------
# buffers
# --------------------------------------------------------------------------

def make_pack_buffers(c: PackCase, rng: np.random.Generator):
    """(input bytes, initial output bytes): both random, sized like
    tools/pack_test.c:88-113 (rows x stride0)."""
    es = c.elem_bytes
    n_in = max(1, c.in_size0 * c.in_stride0)
    n_out = max(1, c.out_size0 * c.out_stride0)
    return (rng.integers(0, 256, n_in * es, dtype=np.uint8),
            rng.integers(0, 256, n_out * es, dtype=np.uint8))


def make_unpack_buffers(c: UnpackCase, rng: np.random.Generator):
    es = c.elem_bytes
    n_in = max(1, c.in_size0 * c.in_stride0)
    n_out = max(1, c.out_size0 * c.out_stride0)
    return (rng.integers(0, 256, n_in * es, dtype=np.uint8),
            rng.integers(0, 256, n_out * es, dtype=np.uint8))


def make_mmt4d_buffers(c: Mmt4dCase, rng: np.random.Generator):
    """(lhs, rhs, out_init) as uint8 byte arrays, rows x stride0 each."""
    lk, rk, ok = MMT4D_KINDS[c.flags & 0xFF]
    lb, rb, ob = c.bits()

    def buf(kind, bits, rows, stride):
        nbytes = max(1, rows * stride * bits // 8)
        n = nbytes if bits == 4 else -(-nbytes * 8 // bits)
        return random_elements(rng, kind, n).view(np.uint8)[:nbytes].copy()

    return (buf(lk, lb, c.M, c.lhs_stride0), buf(rk, rb, c.N, c.rhs_stride0),
            buf(ok, ob, c.M, c.out_stride0))


# --------------------------------------------------------------------------
# numpy formulations used as independent pins
# --------------------------------------------------------------------------

def numpy_pack(x: np.ndarray, tile0: int, tile1: int, transpose_inner: bool,
               transpose_outer: bool, pad) -> np.ndarray:
    """pack as pad + reshape + transpose (tests/e2e/linalg/pack.mlir:96-240;
    docs/website/docs/community/blog/posts/mmt4d.md:190-198). (tile0, tile1)
    is the tile extent along matrix dims 0 and 1. Returns the stored 4-D
    array."""
    s0, s1 = x.shape
    o0, o1 = -(-s0 // tile0), -(-s1 // tile1)
    p = np.full((o0 * tile0, o1 * tile1), pad, dtype=x.dtype)
    p[:s0, :s1] = x
    t = p.reshape(o0, tile0, o1, tile1).transpose(0, 2, 1, 3)  # [a0][a1][b0][b1]
    if transpose_outer:
        t = t.transpose(1, 0, 2, 3)
    if transpose_inner:
        t = t.transpose(0, 1, 3, 2)
    return np.ascontiguousarray(t)


# --------------------------------------------------------------------------
# device helpers (GPU tests only)
# --------------------------------------------------------------------------

class DeviceBytes:
    """A byte buffer in device memory, created from / read back to numpy."""

    def __init__(self, torch, host: np.ndarray):
        self.torch = torch
        flat = np.ascontiguousarray(host).view(np.uint8).reshape(-1)
        self.t = torch.from_numpy(flat.copy()).to("cuda")
        self.ptr = self.t.data_ptr()

    def numpy(self) -> np.ndarray:
        return self.t.cpu().numpy()


def gpu_pack(lib, torch, c: PackCase, inp: np.ndarray, out: np.ndarray) -> np.ndarray:
    """Runs the product pack on device copies of (inp, out); returns the whole
    output buffer as bytes."""
    es = c.elem_bytes
    d_in, d_out = DeviceBytes(torch, inp), DeviceBytes(torch, out)
    lib.pack(d_in.ptr - c.in_offset * es, c.in_offset, c.in_stride0, c.in_stride1,
             d_out.ptr - c.out_offset * es, c.out_offset, c.out_stride0,
             c.out_stride1, c.in_size0, c.in_size1, c.out_size0, c.out_size1,
             c.out_size2, c.out_size3, c.padding_value, c.flags)
    lib.synchronize()
    return d_out.numpy()


def gpu_unpack(lib, torch, c: UnpackCase, inp: np.ndarray, out: np.ndarray) -> np.ndarray:
    es = c.elem_bytes
    d_in, d_out = DeviceBytes(torch, inp), DeviceBytes(torch, out)
    lib.unpack(d_in.ptr - c.in_offset * es, c.in_offset, c.in_stride0, c.in_stride1,
               d_out.ptr - c.out_offset * es, c.out_offset, c.out_stride0,
               c.out_stride1, c.in_size0, c.in_size1, c.in_size2, c.in_size3,
               c.out_size0, c.out_size1, c.flags)
    lib.synchronize()
    return d_out.numpy()


def gpu_mmt4d(lib, torch, c: Mmt4dCase, lhs, rhs, out, allow_generic=True) -> np.ndarray:
    lb, rb, ob = c.bits()
    d_l, d_r, d_o = DeviceBytes(torch, lhs), DeviceBytes(torch, rhs), DeviceBytes(torch, out)
    flags = c.flags | (uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION if allow_generic else 0)
    lib.mmt4d(d_l.ptr - c.lhs_offset * lb // 8, c.lhs_offset, c.lhs_stride0,
              d_r.ptr - c.rhs_offset * rb // 8, c.rhs_offset, c.rhs_stride0,
              d_o.ptr - c.out_offset * ob // 8, c.out_offset, c.out_stride0,
              c.M, c.N, c.K, c.M0, c.N0, c.K0, flags)
    lib.synchronize()
    return d_o.numpy()
