"""Case generation for conv_nchwc, shared by the CPU and GPU tests: the shape
grid and the random strides / offsets of
runtime/src/iree/builtins/ukernel/tools/conv_nchwc_test.c:95-226, plus an
independent numpy statement of the operation."""
import dataclasses

import numpy as np

CONV_TYPE_F32F32F32 = 0x01          # exported_bits.h:115
CONV_ACCUMULATE = 0x100             # exported_bits.h:119
CONV_ALLOW_GENERIC_FALLBACK = 0x200  # exported_bits.h:120

# (N, OC_outer, OH, OW, IC_outer, FH, FW, stride_h, stride_w): conv_nchwc_test.c:187-204
SHAPES = [
    (0, 1, 3, 3, 1, 3, 3, 1, 1), (1, 0, 3, 3, 1, 3, 3, 1, 1), (1, 1, 0, 3, 1, 3, 3, 1, 1),
    (1, 1, 3, 0, 1, 3, 3, 1, 1), (1, 1, 2, 2, 0, 3, 3, 1, 1), (1, 1, 2, 2, 1, 0, 3, 1, 1),
    (1, 1, 2, 2, 1, 3, 0, 1, 1), (1, 1, 1, 1, 1, 1, 1, 1, 1), (1, 1, 1, 15, 1, 1, 1, 1, 1),
    (1, 1, 1, 16, 1, 1, 1, 1, 1), (1, 1, 1, 17, 1, 1, 1, 1, 1), (1, 2, 3, 5, 2, 3, 3, 1, 1),
    (2, 2, 5, 5, 2, 3, 3, 1, 1), (1, 1, 3, 3, 1, 1, 1, 1, 1), (1, 1, 5, 5, 1, 3, 3, 2, 2),
    (1, 1, 1, 33, 1, 3, 3, 1, 1),
]
# (k0, c0): the reference's x86 tile (16, 16) and shapes only a generic path serves.
TILES = [(16, 16), (1, 1), (4, 8), (3, 5), (8, 1)]


@dataclasses.dataclass
class ConvCase:
    N: int
    OC_outer: int
    OH: int
    OW: int
    IC_outer: int
    FH: int
    FW: int
    stride_h: int
    stride_w: int
    k0: int
    c0: int
    flags: int
    in_strides: tuple      # (n, ic_outer, h)
    f_strides: tuple       # (oc_outer, ic_outer, fh)
    out_strides: tuple     # (n, oc_outer, oh)
    offsets: tuple         # (input, filter, output)

    def sizes(self):
        """Element counts of the three buffers (rows x outermost stride, as the
        reference test allocates them), offsets included."""
        return (self.offsets[0] + max(1, self.N * self.in_strides[0]),
                self.offsets[1] + max(1, self.OC_outer * self.f_strides[0]),
                self.offsets[2] + max(1, self.N * self.out_strides[0]))

    def label(self):
        return (f"N{self.N} OC{self.OC_outer} OH{self.OH} OW{self.OW} IC{self.IC_outer} "
                f"F{self.FH}x{self.FW} s{self.stride_h}x{self.stride_w} k0={self.k0} c0={self.c0} "
                f"flags={self.flags:#x} off={self.offsets}")

    def args(self):
        """Positional arguments between the three buffers, in API order."""
        return dict(
            input=(self.offsets[0],) + self.in_strides,
            filter=(self.offsets[1],) + self.f_strides,
            output=(self.offsets[2],) + self.out_strides,
            dims=(self.N, self.OC_outer, self.OH, self.OW, self.IC_outer, self.FH, self.FW,
                  self.k0, self.c0, self.stride_h, self.stride_w, self.flags))


# Larger than anything in the reference's grid: several 16-pixel panels per
# row, an odd number of output-channel blocks, strides in both directions.
WIDE_SHAPES = [(2, 3, 4, 40, 2, 3, 3, 1, 1), (1, 3, 2, 35, 1, 2, 2, 2, 1), (1, 5, 3, 64, 3, 1, 1, 1, 2),
               (1, 2, 2, 17, 1, 3, 3, 2, 2)]


def cases(seed: int, tiles=None, shapes=None):
    rng = np.random.default_rng(seed)
    for (k0, c0) in (tiles or TILES):
        for shape in (shapes or SHAPES):
            for acc in (0, 1):
                N, OC, OH, OW, IC, FH, FW, sh, sw = shape
                H = (OH - 1) * sh + FH if OH else FH
                W = (OW - 1) * sw + FW if OW else FW
                bit = lambda: int(rng.integers(0, 2))
                ish = W * c0 + bit()
                isic = H * ish + bit()
                isn = IC * isic + bit()
                fsfh = FW * c0 * k0 + bit()
                fsic = FH * fsfh + bit()
                fsoc = IC * fsic + bit()
                osoh = OW * k0 + bit()
                osoc = OH * osoh + bit()
                osn = OC * osoc + bit()
                yield ConvCase(N, OC, OH, OW, IC, FH, FW, sh, sw, k0, c0,
                               CONV_TYPE_F32F32F32 | CONV_ALLOW_GENERIC_FALLBACK |
                               (CONV_ACCUMULATE if acc else 0),
                               (isn, isic, ish), (fsoc, fsic, fsfh), (osn, osoc, osoh),
                               (bit(), bit(), bit()))


def buffers(c: ConvCase, rng: np.random.Generator, exact: bool = True):
    """(input, filter, output_init) as float32 arrays. exact: small integers,
    as the reference's tests use (tools/util.c:137-147), so that any summation
    order gives the same bits."""
    n_in, n_f, n_out = c.sizes()
    if exact:
        gen = lambda n: rng.integers(-8, 9, n).astype(np.float32)
    else:
        gen = lambda n: rng.standard_normal(n).astype(np.float32)
    return gen(n_in), gen(n_f), gen(n_out)


def run(chk, c: ConvCase, inp, flt, out):
    a = c.args()
    chk.conv_nchwc(inp, *a["input"], flt, *a["filter"], out, *a["output"], *a["dims"][:7],
                   *a["dims"][7:])


def numpy_conv(c: ConvCase, inp, flt, out):
    """The operation written independently of the ukernel's loop nest: gather
    the dense tensors through the strides, one einsum per (fh, fw), f64
    accumulation; returns the dense [N][OC][OH][OW][k0] result (f64)."""
    (io, fo, oo) = c.offsets
    H = (c.OH - 1) * c.stride_h + c.FH
    W = (c.OW - 1) * c.stride_w + c.FW
    x = np.zeros((c.N, c.IC_outer, H, W, c.c0))
    for n in range(c.N):
        for ic in range(c.IC_outer):
            for h in range(H):
                base = io + n * c.in_strides[0] + ic * c.in_strides[1] + h * c.in_strides[2]
                x[n, ic, h] = inp[base:base + W * c.c0].reshape(W, c.c0)
    w = np.zeros((c.OC_outer, c.IC_outer, c.FH, c.FW, c.c0, c.k0))
    for oc in range(c.OC_outer):
        for ic in range(c.IC_outer):
            for fh in range(c.FH):
                base = fo + oc * c.f_strides[0] + ic * c.f_strides[1] + fh * c.f_strides[2]
                w[oc, ic, fh] = flt[base:base + c.FW * c.c0 * c.k0].reshape(c.FW, c.c0, c.k0)
    y = np.zeros((c.N, c.OC_outer, c.OH, c.OW, c.k0))
    if c.flags & CONV_ACCUMULATE:
        for n in range(c.N):
            for oc in range(c.OC_outer):
                for oh in range(c.OH):
                    base = oo + n * c.out_strides[0] + oc * c.out_strides[1] + oh * c.out_strides[2]
                    y[n, oc, oh] = out[base:base + c.OW * c.k0].reshape(c.OW, c.k0)
    for fh in range(c.FH):
        for fw in range(c.FW):
            xs = x[:, :, fh:fh + (c.OH - 1) * c.stride_h + 1:c.stride_h,
                   fw:fw + (c.OW - 1) * c.stride_w + 1:c.stride_w, :]
            y += np.einsum("nihwc,oick->nohwk", xs, w[:, :, fh, fw])
    return y


def dense_output(c: ConvCase, out):
    oo = c.offsets[2]
    y = np.zeros((c.N, c.OC_outer, c.OH, c.OW, c.k0), np.float32)
    for n in range(c.N):
        for oc in range(c.OC_outer):
            for oh in range(c.OH):
                base = oo + n * c.out_strides[0] + oc * c.out_strides[1] + oh * c.out_strides[2]
                y[n, oc, oh] = out[base:base + c.OW * c.k0].reshape(c.OW, c.k0)
    return y
