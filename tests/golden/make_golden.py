"""Writes the golden fixtures of tests/golden/ by running the compiled
reference C ukernels (oracle/_ref/libiree_uk_ref.so, built from the reference
checkout by oracle/Makefile). Run from the repository root in a container that
has the reference:

    make -C oracle all && python tests/golden/make_golden.py

Fixtures (data only):
  reference_kat.json   small known-answer vectors (inputs and outputs);
  reference_sweep.json SHA-256 digests of the reference's output buffers over
                       a seeded sweep shaped like the reference's own unit
                       tests (tools/{pack,unpack,mmt4d}_test.c); the inputs
                       are regenerated from the seeds by `sweep_digests`.
"""
from __future__ import annotations

import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
TESTS = os.path.dirname(HERE)
ROOT = os.path.dirname(TESTS)
for p in (ROOT, TESTS):
    if p not in sys.path:
        sys.path.insert(0, p)

import uk_testing as T  # noqa: E402
from iree_amd import ukernel as uk  # noqa: E402

# (type flag, tile) lists of the reference's generic test cases
# (tools/pack_test.c:215-219, unpack_test.c:202-205, mmt4d_test.c:550-559) plus
# the tile shapes of the benchmark configurations.
PACK_TILES = [(uk.PACK_TYPE_F32F32, 3, 5), (uk.PACK_TYPE_I8I8, 4, 2),
              (uk.PACK_TYPE_I32I32, 3, 4), (uk.PACK_TYPE_F16F16, 6, 7),
              (uk.PACK_TYPE_BF16BF16, 9, 2), (uk.PACK_TYPE_F16F16, 16, 16),
              (uk.PACK_TYPE_I8I8, 16, 32), (uk.PACK_TYPE_F32F32, 16, 1),
              (uk.PACK_TYPE_I8I8, 16, 2), (uk.PACK_TYPE_I8I8, 32, 8)]
UNPACK_TILES = [(uk.UNPACK_TYPE_F32F32, 3, 5), (uk.UNPACK_TYPE_I32I32, 3, 4),
                (uk.UNPACK_TYPE_F16F16, 6, 7), (uk.UNPACK_TYPE_BF16BF16, 9, 2),
                (uk.UNPACK_TYPE_F32F32, 16, 16), (uk.UNPACK_TYPE_F32F32, 16, 1),
                (uk.UNPACK_TYPE_I32I32, 32, 16)]
MMT4D_TILES = [(uk.MMT4D_TYPE_F32F32F32, 3, 5, 7, 0), (uk.MMT4D_TYPE_S8S8S32, 9, 6, 3, 0),
               (uk.MMT4D_TYPE_S8S4S32, 9, 12, 2, 0), (uk.MMT4D_TYPE_S16S16S32, 7, 3, 6, 0),
               (uk.MMT4D_TYPE_S16U4S32, 5, 3, 2, 0), (uk.MMT4D_TYPE_S16S8S32, 7, 5, 6, 0),
               (uk.MMT4D_TYPE_F16F16F32, 4, 6, 5, 0), (uk.MMT4D_TYPE_F16F16F16, 3, 5, 8, 0),
               (uk.MMT4D_TYPE_F16F16F16, 3, 5, 8, uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS),
               (uk.MMT4D_TYPE_BF16BF16F32, 11, 4, 1, 0), (uk.MMT4D_TYPE_BF16BF16BF16, 2, 9, 3, 0),
               (uk.MMT4D_TYPE_BF16BF16BF16, 2, 9, 3, uk.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS),
               (uk.MMT4D_TYPE_S8S8S32, 16, 16, 2, 0), (uk.MMT4D_TYPE_S8S8S32, 32, 16, 8, 0),
               (uk.MMT4D_TYPE_F16F16F32, 16, 16, 16, 0), (uk.MMT4D_TYPE_BF16BF16F32, 16, 16, 2, 0)]


def run_pack_case(chk, c: T.PackCase, inp: np.ndarray, out: np.ndarray):
    es = c.elem_bytes
    chk.pack(inp, c.in_offset, c.in_stride0, c.in_stride1, out, c.out_offset,
             c.out_stride0, c.out_stride1, c.in_size0, c.in_size1, c.out_size0,
             c.out_size1, c.out_size2, c.out_size3, c.padding_value, c.flags,
             in_shift=-c.in_offset * es, out_shift=-c.out_offset * es)


def run_unpack_case(chk, c: T.UnpackCase, inp: np.ndarray, out: np.ndarray):
    es = c.elem_bytes
    chk.unpack(inp, c.in_offset, c.in_stride0, c.in_stride1, out, c.out_offset,
               c.out_stride0, c.out_stride1, c.in_size0, c.in_size1, c.in_size2,
               c.in_size3, c.out_size0, c.out_size1, c.flags,
               in_shift=-c.in_offset * es, out_shift=-c.out_offset * es)


def run_mmt4d_case(chk, c: T.Mmt4dCase, lhs, rhs, out):
    lb, rb, ob = c.bits()
    chk.mmt4d(lhs, c.lhs_offset, c.lhs_stride0, rhs, c.rhs_offset, c.rhs_stride0,
              out, c.out_offset, c.out_stride0, c.M, c.N, c.K, c.M0, c.N0, c.K0,
              c.flags | uk.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION,
              lhs_shift=-c.lhs_offset * lb // 8, rhs_shift=-c.rhs_offset * rb // 8,
              out_shift=-c.out_offset * ob // 8)


def _digest(buf: np.ndarray) -> str:
    return hashlib.sha256(buf.tobytes()).hexdigest()[:20]


def sweep_digests(chk) -> dict:
    """case id -> leading 80 bits of the SHA-256 of the whole output buffer (stride gaps included) for
    every case of the seeded sweep, computed with checker `chk`."""
    digests = {}
    for n, (tf, t0, t1) in enumerate(PACK_TILES):
        for ci, c in enumerate(T.pack_cases(tf, t0, t1, seed=100 + n)):
            rng = np.random.default_rng(1000 * n + ci)
            inp, out = T.make_pack_buffers(c, rng)
            run_pack_case(chk, c, inp, out)
            digests[f"pack/{n}/{ci}"] = _digest(out)
    for n, (tf, t0, t1) in enumerate(UNPACK_TILES):
        for ci, c in enumerate(T.unpack_cases(tf, t0, t1, seed=200 + n)):
            rng = np.random.default_rng(50000 + 1000 * n + ci)
            inp, out = T.make_unpack_buffers(c, rng)
            run_unpack_case(chk, c, inp, out)
            digests[f"unpack/{n}/{ci}"] = _digest(out)
    for n, (tf, M0, N0, K0, extra) in enumerate(MMT4D_TILES):
        for ci, c in enumerate(T.mmt4d_cases(tf, M0, N0, K0, seed=300 + n, extra_flags=extra)):
            rng = np.random.default_rng(90000 + 1000 * n + ci)
            lhs, rhs, out = T.make_mmt4d_buffers(c, rng)
            run_mmt4d_case(chk, c, lhs, rhs, out)
            digests[f"mmt4d/{n}/{ci}"] = _digest(out)
    return digests


def conv_digests(chk) -> dict:
    """case index -> digest of the whole output buffer for the seeded conv_nchwc
    sweep (small-integer and N(0,1) inputs), computed with checker `chk`."""
    import conv_testing as C
    digests = {}
    for ci, c in enumerate(C.cases(seed=31)):
        for exact in (True, False):
            rng = np.random.default_rng(7000 + ci)
            inp, flt, out = C.buffers(c, rng, exact=exact)
            C.run(chk, c, inp, flt, out)
            digests[f"conv/{ci}/{int(exact)}"] = _digest(out)
    return digests


def known_answers(ref) -> dict:
    kat = {"pack": [], "unpack": [], "mmt4d_s8": []}
    x = np.array([[10 * i + j for j in range(5)] for i in range(3)], dtype=np.int8)
    for flags, (o0, o1) in ((0x002, (2, 2)), (0x102, (1, 3)), (0x202, (2, 2)), (0x302, (3, 1))):
        out = np.full(o0 * o1 * 6, 99, dtype=np.int8)
        ref.pack(x, 0, 5, 1, out, 0, o1 * 6, 6, 3, 5, o0, o1, 2, 3, 0xEE, flags)
        kat["pack"].append({"flags": flags, "in": x.ravel().tolist(),
                            "out_size01": [o0, o1], "out": out.tolist()})
    for flags, (i0, i1) in ((0x003, (2, 2)), (0x103, (1, 3)), (0x203, (2, 2)), (0x303, (3, 1))):
        inp = np.arange(i0 * i1 * 6, dtype=np.int32)
        out = np.full(15, -1, dtype=np.int32)
        ref.unpack(inp, 0, i1 * 6, 6, out, 0, 5, 1, i0, i1, 2, 3, 3, 5, flags)
        kat["unpack"].append({"flags": flags, "in_size01": [i0, i1], "out": out.tolist()})
    lhs = np.array([1, 2, 3, 4, 5, 6, 7, 8], dtype=np.int8)
    rhs = np.array([1, 0, 0, 1, -1, 2, 3, -4], dtype=np.int8)
    for flags in (0x202, 0x302):
        out = np.array([100, 200, 300, 400], dtype=np.int32)
        ref.mmt4d(lhs, 0, 8, rhs, 0, 8, out, 0, 4, 1, 1, 2, 2, 2, 2, flags)
        kat["mmt4d_s8"].append({"flags": flags, "lhs": lhs.tolist(), "rhs": rhs.tolist(),
                                "out_init": [100, 200, 300, 400], "out": out.tolist()})
    l16 = np.array([0x0001, 0x3C00], dtype=np.uint16)
    r16 = np.array([0x7BFF, 0x4000], dtype=np.uint16)
    o = np.zeros(1, dtype=np.float32)
    ref.mmt4d(l16, 0, 2, r16, 0, 2, o, 0, 1, 1, 1, 1, 1, 1, 2, 0x203)
    kat["mmt4d_f16_flush"] = {"lhs": l16.tolist(), "rhs": r16.tolist(), "out": float(o[0])}
    return kat


def main():
    from oracle import uk_oracle
    ref = uk_oracle.get("reference")  # cpu_data all zero: generic code paths
    with open(os.path.join(HERE, "reference_kat.json"), "w") as f:
        json.dump(known_answers(ref), f, indent=1)
    with open(os.path.join(HERE, "reference_sweep.json"), "w") as f:
        json.dump(sweep_digests(ref), f, indent=0, sort_keys=True)
    with open(os.path.join(HERE, "reference_conv.json"), "w") as f:
        json.dump(conv_digests(ref), f, indent=0, sort_keys=True)
    print("wrote reference_kat.json, reference_sweep.json, reference_conv.json")


if __name__ == "__main__":
    main()
