/*
 * CPU oracle for the pack / mmt4d / unpack ukernels.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. Only tests, the smoke check
 * and the benchmark's cpu_baseline leg may load it; the shipped library never
 * links, loads or calls anything in this directory.
 *
 * It restates, in plain scalar C, the arithmetic that the reference CPU
 * ukernels define (paths relative to the reference checkout):
 *   mmt4d : runtime/src/iree/builtins/ukernel/mmt4d.c:55-114 (outer loops,
 *           early-outs) and mmt4d_tile_generic.c:11-376 (one loop nest per
 *           type triple; this file is the arithmetic definition);
 *   pack  : runtime/src/iree/builtins/ukernel/pack.c:254-323 and the 4-loop
 *           definition in tools/pack_test.c:13-71;
 *   unpack: runtime/src/iree/builtins/ukernel/unpack.c:190-257 and
 *           tools/unpack_test.c:13-58;
 *   f16/bf16 <-> f32: runtime/src/iree/builtins/ukernel/common.h:665-792;
 *   f8E4M3FN -> f32 : runtime/src/iree/base/internal/math.h:324-362,557-560;
 *   f8 matmul       : tools/testing/e2e/iree-e2e-matmul-test.cc:123-142
 *                     (decode both operands, accumulate sequentially in f32);
 *   conv_nchwc      : runtime/src/iree/builtins/ukernel/conv_nchwc.c:42-130
 *                     (early-outs, pointer arithmetic) and
 *                     conv_nchwc_tile_generic.c:11-61 (the loop nest).
 *
 * Pinning status (what each function is checked against, in tests/):
 *   uk_oracle_pack / uk_oracle_unpack : golden tensors of
 *       tests/e2e/linalg/{pack,unpack}.mlir, known-answer vectors produced by
 *       the reference build, reshape+transpose identities, round trips, and
 *       randomized sweeps against the compiled reference (oracle/_ref).
 *   uk_oracle_mmt4d (all upstream type triples) : known-answer vectors,
 *       brute-force row-major matmul on unpacked operands, ACCUMULATE / K==0
 *       invariants, randomized sweeps against the compiled reference.
 *   uk_oracle_f8e4m3fn_to_f32 : all 256 encodings against the closed form
 *       and the conversion known-answer values of
 *       runtime/src/iree/base/internal/math_test.cc:483-589.
 *   uk_oracle_mmt4d with the f8 type : the reference has no f8 ukernel; the
 *       function is pinned by the decode table plus the f32 loop above, and
 *       by exactness on inputs whose products and sums are exact in f32.
 *
 *   uk_oracle_conv_nchwc : the independent per-pixel definition of
 *       tools/conv_nchwc_test.c:13-87 restated in numpy (tests), a direct
 *       convolution closed form on dense tensors, and randomized sweeps
 *       against the compiled reference (oracle/_ref).
 *
 * Compile with -ffp-contract=off so that `acc += a*b` is a separate multiply
 * and add, which is what the reference generic build does on baseline x86-64.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define UK_ORACLE_EXPORT __attribute__((visibility("default")))

/* Flag values: runtime/src/iree/builtins/ukernel/exported_bits.h:29-83. */
enum {
  kTypeMask = 0xFF,
  kMmt4dF32F32F32 = 0x01,
  kMmt4dS8S8S32 = 0x02,
  kMmt4dF16F16F32 = 0x03,
  kMmt4dF16F16F16 = 0x04,
  kMmt4dBF16BF16F32 = 0x05,
  kMmt4dBF16BF16BF16 = 0x06,
  kMmt4dS16S16S32 = 0x07,
  kMmt4dS16U4S32 = 0x08,
  kMmt4dS16S8S32 = 0x09,
  kMmt4dS8S4S32 = 0x0A,
  kMmt4dF8F8F32 = 0x80, /* extension, not upstream */
  kMmt4dAccumulate = 0x100,
  kMmt4dSkipRoundings = 0x400,
  kPackF32 = 0x01,
  kPackI8 = 0x02,
  kPackI32 = 0x03,
  kPackF16 = 0x04,
  kPackBF16 = 0x05,
  kTransposeInner = 0x100,
  kTransposeOuter = 0x200,
};

/* When non-zero (the default, = reference behaviour) f16/bf16 inputs with a
 * zero exponent field decode to +-0 (common.h:685-686). */
static int g_flush_subnormal_inputs = 1;

UK_ORACLE_EXPORT void uk_oracle_set_flush_subnormal_inputs(int on) {
  g_flush_subnormal_inputs = on;
}

/*---------------------------------------------------------------------------
 * Small-float conversions.
 *-------------------------------------------------------------------------*/

static float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

static uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  return u;
}

/* 16-bit float with `ebits` exponent bits -> f32 (common.h:665-699).
 * Inf stays Inf, any NaN becomes a quiet NaN with an all-ones mantissa,
 * exponent field 0 (zero AND subnormals) becomes a signed zero. */
static float small16_to_f32(uint16_t v, int ebits) {
  const int mbits = 15 - ebits;
  const uint32_t sign = (uint32_t)(v >> 15) << 31;
  const uint32_t e = (v >> mbits) & ((1u << ebits) - 1);
  const uint32_t m = v & ((1u << mbits) - 1);
  if (e == (1u << ebits) - 1) {
    return bits_to_f32(sign | 0x7F800000u | (m ? 0x007FFFFFu : 0u));
  }
  if (e == 0) {
    if (g_flush_subnormal_inputs || m == 0) return bits_to_f32(sign);
    /* IEEE value of the subnormal (only when the flush is switched off). */
    float mag = ldexpf((float)m, 1 - ((1 << (ebits - 1)) - 1) - mbits);
    return (v >> 15) ? -mag : mag;
  }
  const uint32_t e32 = e + 128u - (1u << (ebits - 1)); /* rebias 2^(e-1)-1 -> 127 */
  return bits_to_f32(sign | (e32 << 23) | (m << (23 - mbits)));
}

UK_ORACLE_EXPORT float uk_oracle_f16_to_f32(uint16_t v) {
  return small16_to_f32(v, 5);
}
UK_ORACLE_EXPORT float uk_oracle_bf16_to_f32(uint16_t v) {
  return small16_to_f32(v, 8);
}

/* f32 -> 16-bit float with `ebits` exponent bits, round to nearest even
 * (common.h:701-770). The upstream routine measures the exponent against 128
 * rather than 127, which makes its overflow/underflow tests one binade late:
 * inputs with unbiased exponent 2^(ebits-1) come out with an all-ones
 * exponent field, and inputs with the smallest normal exponent minus one come
 * out with exponent field 0 and their mantissa bits kept. f32 subnormal
 * inputs give zero. Restated as is, because f16/bf16 *outputs* of the
 * reference are defined by it. */
static uint16_t f32_to_small16(float value, int ebits) {
  const int mbits = 15 - ebits;
  const uint32_t u = f32_to_bits(value);
  const uint32_t sign16 = (u >> 31) << 15;
  const uint32_t e32 = (u >> 23) & 0xFF;
  const uint32_t m32 = u & 0x007FFFFFu;
  const uint32_t emask16 = ((1u << ebits) - 1) << mbits;
  const uint32_t mmask16 = (1u << mbits) - 1;
  if (e32 == 0xFF) return (uint16_t)(sign16 | emask16 | (m32 ? mmask16 : 0));
  if (e32 == 0) return (uint16_t)sign16;
  int ex = (int)e32 - 128;
  const int half_range = 1 << (ebits - 1);
  if (ex >= half_range) return (uint16_t)(sign16 | emask16);
  if (ex < -half_range) return (uint16_t)sign16;
  const int drop = 23 - mbits;
  const uint32_t even_bit = 1u << drop;
  const uint32_t odd_bit = even_bit >> 1;
  uint32_t biased = m32 + ((m32 & even_bit) ? odd_bit : odd_bit - 1);
  if (biased > 0x007FFFFFu) {
    biased = 0;
    ++ex;
  }
  const uint32_t e16 = (uint32_t)(ex + half_range) << mbits;
  return (uint16_t)(sign16 | e16 | (biased >> drop));
}

UK_ORACLE_EXPORT uint16_t uk_oracle_f32_to_f16(float v) {
  return f32_to_small16(v, 5);
}
UK_ORACLE_EXPORT uint16_t uk_oracle_f32_to_bf16(float v) {
  return f32_to_small16(v, 8);
}

/* f8E4M3FN -> f32 (math.h:324-362 with exp_bits=4, mantissa_bits=3,
 * have_infinity=false, have_nan=true, bias 7): S.1111.111 is NaN (returned as
 * the positive quiet NaN of <math.h>), exponent field 0 is a kept subnormal
 * m * 2^-9, everything else (1 + m/8) * 2^(e-7), up to 448. */
UK_ORACLE_EXPORT float uk_oracle_f8e4m3fn_to_f32(uint8_t v) {
  const float sign = (v & 0x80) ? -1.f : 1.f;
  const int e = (v >> 3) & 0xF;
  const int m = v & 0x7;
  if (e == 0xF && m == 0x7) return NAN;
  if (e == 0) return sign * ldexpf((float)m, 1 - 7 - 3);
  return sign * ldexpf((float)(m + 8), e - 7 - 3);
}

/*---------------------------------------------------------------------------
 * mmt4d.
 *-------------------------------------------------------------------------*/

typedef struct {
  int lhs_bits, rhs_bits, out_bytes;
} type_sizes_t;

static int mmt4d_type_sizes(uint32_t flags, type_sizes_t* s) {
  switch (flags & kTypeMask) {
    case kMmt4dF32F32F32: *s = (type_sizes_t){32, 32, 4}; return 1;
    case kMmt4dS8S8S32: *s = (type_sizes_t){8, 8, 4}; return 1;
    case kMmt4dF16F16F32: *s = (type_sizes_t){16, 16, 4}; return 1;
    case kMmt4dF16F16F16: *s = (type_sizes_t){16, 16, 2}; return 1;
    case kMmt4dBF16BF16F32: *s = (type_sizes_t){16, 16, 4}; return 1;
    case kMmt4dBF16BF16BF16: *s = (type_sizes_t){16, 16, 2}; return 1;
    case kMmt4dS16S16S32: *s = (type_sizes_t){16, 16, 4}; return 1;
    case kMmt4dS16U4S32: *s = (type_sizes_t){16, 4, 4}; return 1;
    case kMmt4dS16S8S32: *s = (type_sizes_t){16, 8, 4}; return 1;
    case kMmt4dS8S4S32: *s = (type_sizes_t){8, 4, 4}; return 1;
    case kMmt4dF8F8F32: *s = (type_sizes_t){8, 8, 4}; return 1;
    default: return 0;
  }
}

/* One M0xN0 tile: out[i0][j0] = (acc? out : 0) + sum_k sum_k0 l*r, with the
 * (k, k0) order and per-type conversions of mmt4d_tile_generic.c. The lhs
 * panel is [K][M0][K0], the rhs panel [K][N0][K0]. */
static void mmt4d_tile(void* out_tile, const void* lhs_panel,
                       const void* rhs_panel, int64_t K, int M0, int N0,
                       int K0, uint32_t flags) {
  const int accumulate = (flags & kMmt4dAccumulate) != 0;
  const int skip_round = (flags & kMmt4dSkipRoundings) != 0;
  const uint32_t type = flags & kTypeMask;
  for (int i0 = 0; i0 < M0; ++i0) {
    for (int j0 = 0; j0 < N0; ++j0) {
      const int64_t o = (int64_t)i0 * N0 + j0;
      switch (type) {
        case kMmt4dS8S8S32:   /* mmt4d_tile_generic.c:54-78 */
        case kMmt4dS16S16S32: /* :81-105 */
        case kMmt4dS16S8S32: {/* :145-169 */
          int32_t* out = (int32_t*)out_tile;
          /* Accumulate modulo 2^32 (the reference relies on wrapping int32). */
          uint32_t acc = accumulate ? (uint32_t)out[o] : 0u;
          for (int64_t k = 0; k < K; ++k) {
            for (int k0 = 0; k0 < K0; ++k0) {
              const int64_t li = (k * M0 + i0) * K0 + k0;
              const int64_t ri = (k * N0 + j0) * K0 + k0;
              int32_t l = (type == kMmt4dS8S8S32)
                              ? ((const int8_t*)lhs_panel)[li]
                              : ((const int16_t*)lhs_panel)[li];
              int32_t r = (type == kMmt4dS16S16S32)
                              ? ((const int16_t*)rhs_panel)[ri]
                              : ((const int8_t*)rhs_panel)[ri];
              acc += (uint32_t)(l * r);
            }
          }
          out[o] = (int32_t)acc;
          break;
        }
        case kMmt4dS8S4S32:   /* :11-51: two signed nibbles per rhs byte, low first */
        case kMmt4dS16U4S32: {/* :108-142: two unsigned nibbles per rhs byte */
          int32_t* out = (int32_t*)out_tile;
          uint32_t acc = accumulate ? (uint32_t)out[o] : 0u;
          const int K0half = K0 / 2;
          const uint8_t* rhs = (const uint8_t*)rhs_panel;
          for (int64_t k = 0; k < K; ++k) {
            for (int h = 0; h < K0half; ++h) {
              const int64_t li = (k * M0 + i0) * K0 + 2 * h;
              int32_t l0, l1;
              if (type == kMmt4dS8S4S32) {
                l0 = ((const int8_t*)lhs_panel)[li];
                l1 = ((const int8_t*)lhs_panel)[li + 1];
              } else {
                l0 = ((const int16_t*)lhs_panel)[li];
                l1 = ((const int16_t*)lhs_panel)[li + 1];
              }
              const uint8_t byte = rhs[(k * N0 + j0) * K0half + h];
              int32_t r0 = byte & 0xF, r1 = byte >> 4;
              if (type == kMmt4dS8S4S32) {
                if (r0 & 8) r0 -= 16;
                if (r1 & 8) r1 -= 16;
              }
              acc += (uint32_t)(l0 * r0 + l1 * r1);
            }
          }
          out[o] = (int32_t)acc;
          break;
        }
        case kMmt4dF32F32F32: { /* :172-196 */
          float* out = (float*)out_tile;
          float acc = accumulate ? out[o] : 0.f;
          const float* l = (const float*)lhs_panel;
          const float* r = (const float*)rhs_panel;
          for (int64_t k = 0; k < K; ++k)
            for (int k0 = 0; k0 < K0; ++k0)
              acc += l[(k * M0 + i0) * K0 + k0] * r[(k * N0 + j0) * K0 + k0];
          out[o] = acc;
          break;
        }
        case kMmt4dF16F16F32:     /* :199-225 */
        case kMmt4dBF16BF16F32: { /* :289-315 */
          const int eb = (type == kMmt4dF16F16F32) ? 5 : 8;
          float* out = (float*)out_tile;
          float acc = accumulate ? out[o] : 0.f;
          const uint16_t* l = (const uint16_t*)lhs_panel;
          const uint16_t* r = (const uint16_t*)rhs_panel;
          for (int64_t k = 0; k < K; ++k)
            for (int k0 = 0; k0 < K0; ++k0)
              acc += small16_to_f32(l[(k * M0 + i0) * K0 + k0], eb) *
                     small16_to_f32(r[(k * N0 + j0) * K0 + k0], eb);
          out[o] = acc;
          break;
        }
        case kMmt4dF16F16F16:      /* :229-286 */
        case kMmt4dBF16BF16BF16: { /* :319-376 */
          const int eb = (type == kMmt4dF16F16F16) ? 5 : 8;
          uint16_t* out = (uint16_t*)out_tile;
          const uint16_t* l = (const uint16_t*)lhs_panel;
          const uint16_t* r = (const uint16_t*)rhs_panel;
          if (skip_round) {
            float acc = accumulate ? small16_to_f32(out[o], eb) : 0.f;
            for (int64_t k = 0; k < K; ++k)
              for (int k0 = 0; k0 < K0; ++k0)
                acc += small16_to_f32(l[(k * M0 + i0) * K0 + k0], eb) *
                       small16_to_f32(r[(k * N0 + j0) * K0 + k0], eb);
            out[o] = f32_to_small16(acc, eb);
          } else {
            /* The running sum is rounded to the 16-bit type after every
             * multiply-add. */
            uint16_t acc = accumulate ? out[o] : 0;
            for (int64_t k = 0; k < K; ++k)
              for (int k0 = 0; k0 < K0; ++k0) {
                float a = small16_to_f32(l[(k * M0 + i0) * K0 + k0], eb);
                float b = small16_to_f32(r[(k * N0 + j0) * K0 + k0], eb);
                acc = f32_to_small16(small16_to_f32(acc, eb) + a * b, eb);
              }
            out[o] = acc;
          }
          break;
        }
        case kMmt4dF8F8F32: { /* iree-e2e-matmul-test.cc:123-139 */
          float* out = (float*)out_tile;
          float acc = accumulate ? out[o] : 0.f;
          const uint8_t* l = (const uint8_t*)lhs_panel;
          const uint8_t* r = (const uint8_t*)rhs_panel;
          for (int64_t k = 0; k < K; ++k)
            for (int k0 = 0; k0 < K0; ++k0)
              acc += uk_oracle_f8e4m3fn_to_f32(l[(k * M0 + i0) * K0 + k0]) *
                     uk_oracle_f8e4m3fn_to_f32(r[(k * N0 + j0) * K0 + k0]);
          out[o] = acc;
          break;
        }
        default:
          return;
      }
    }
  }
}

/* Same argument list as iree_uk_mmt4d (mmt4d.h:14-21). Returns 0, or -1 for an
 * unknown type. Offsets and strides are in elements; sub-byte rhs types
 * convert through bits (mmt4d.c:70-83). */
UK_ORACLE_EXPORT int uk_oracle_mmt4d(
    const void* lhs_buffer, int64_t lhs_offset, int64_t lhs_stride0,
    const void* rhs_buffer, int64_t rhs_offset, int64_t rhs_stride0,
    void* out_buffer, int64_t out_offset, int64_t out_stride0, int64_t M,
    int64_t N, int64_t K, int32_t M0, int32_t N0, int32_t K0, uint32_t flags,
    const uint64_t* cpu_data) {
  (void)cpu_data;
  type_sizes_t ts;
  if (!mmt4d_type_sizes(flags, &ts)) return -1;
  /* mmt4d.c:106-114 */
  if (M == 0 || N == 0 || (K == 0 && (flags & kMmt4dAccumulate))) return 0;
  const char* lhs = (const char*)lhs_buffer + lhs_offset * ts.lhs_bits / 8;
  const char* rhs = (const char*)rhs_buffer + rhs_offset * ts.rhs_bits / 8;
  char* out = (char*)out_buffer + out_offset * ts.out_bytes;
  const int64_t lhs_step = lhs_stride0 * ts.lhs_bits / 8;
  const int64_t rhs_step = rhs_stride0 * ts.rhs_bits / 8;
  const int64_t out_step = out_stride0 * ts.out_bytes;
  const int64_t out_tile_bytes = (int64_t)M0 * N0 * ts.out_bytes;
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      mmt4d_tile(out + i * out_step + j * out_tile_bytes, lhs + i * lhs_step,
                 rhs + j * rhs_step, K, M0, N0, K0, flags);
    }
  }
  return 0;
}

/*---------------------------------------------------------------------------
 * pack / unpack.
 *-------------------------------------------------------------------------*/

static int pack_elem_size(uint32_t flags) {
  switch (flags & kTypeMask) {
    case kPackF32: return 4;
    case kPackI8: return 1;
    case kPackI32: return 4;
    case kPackF16: return 2;
    case kPackBF16: return 2;
    default: return 0;
  }
}

static void swap_i64(int64_t* a, int64_t* b) {
  int64_t t = *a;
  *a = *b;
  *b = t;
}

/* Same argument list as iree_uk_pack (pack.h:26-34). Element map
 * (tools/pack_test.c:13-71): with (outer0,outer1,tile0,tile1) the 4-D output
 * shape after undoing the transposes, source element
 * (a0*tile0+b0, a1*tile1+b1) lands at
 * out_offset + a0*sl0 + a1*sl1 + b0*sl2 + b1*sl3, padding where the source
 * index is out of range. */
UK_ORACLE_EXPORT int uk_oracle_pack(
    const void* in_buffer, int64_t in_offset, int64_t in_stride0,
    int64_t in_stride1, void* out_buffer, int64_t out_offset,
    int64_t out_stride0, int64_t out_stride1, int64_t in_size0,
    int64_t in_size1, int64_t out_size0, int64_t out_size1, int64_t out_size2,
    int64_t out_size3, uint64_t padding_value, uint32_t flags,
    const uint64_t* cpu_data) {
  (void)cpu_data;
  (void)out_stride1; /* contract: equals out_size2*out_size3 (pack.c:72) */
  const int es = pack_elem_size(flags);
  if (!es) return -1;
  /* pack.c:106-109 */
  if (!out_size0 || !out_size1 || !out_size2 || !out_size3) return 0;
  int64_t outer0 = out_size0, outer1 = out_size1;
  int64_t tile0 = out_size2, tile1 = out_size3;
  int64_t sl0 = out_stride0, sl1 = out_size2 * out_size3;
  int64_t sl2 = out_size3, sl3 = 1;
  if (flags & kTransposeOuter) {
    swap_i64(&outer0, &outer1);
    swap_i64(&sl0, &sl1);
  }
  if (flags & kTransposeInner) {
    swap_i64(&tile0, &tile1);
    swap_i64(&sl2, &sl3);
  }
  const char* in = (const char*)in_buffer;
  char* out = (char*)out_buffer;
  for (int64_t a0 = 0; a0 < outer0; ++a0)
    for (int64_t a1 = 0; a1 < outer1; ++a1)
      for (int64_t b0 = 0; b0 < tile0; ++b0)
        for (int64_t b1 = 0; b1 < tile1; ++b1) {
          const int64_t i0 = a0 * tile0 + b0, i1 = a1 * tile1 + b1;
          char* dst =
              out + (out_offset + a0 * sl0 + a1 * sl1 + b0 * sl2 + b1 * sl3) * es;
          if (i0 < in_size0 && i1 < in_size1) {
            memcpy(dst, in + (in_offset + i0 * in_stride0 + i1 * in_stride1) * es,
                   es);
          } else {
            /* low `es` bytes of the little-endian padding value (pack.h:16-25) */
            memcpy(dst, &padding_value, es);
          }
        }
  return 0;
}

/* Same argument list as iree_uk_unpack (unpack.h:17-25); inverse map of pack
 * without padding (tools/unpack_test.c:13-58). */
UK_ORACLE_EXPORT int uk_oracle_unpack(
    const void* in_buffer, int64_t in_offset, int64_t in_stride0,
    int64_t in_stride1, void* out_buffer, int64_t out_offset,
    int64_t out_stride0, int64_t out_stride1, int64_t in_size0,
    int64_t in_size1, int64_t in_size2, int64_t in_size3, int64_t out_size0,
    int64_t out_size1, uint32_t flags, const uint64_t* cpu_data) {
  (void)cpu_data;
  (void)in_stride1; /* contract: equals in_size2*in_size3 (unpack.c:49) */
  const int es = pack_elem_size(flags);
  if (!es) return -1;
  /* unpack.c:84-86 */
  if (!out_size0 || !out_size1) return 0;
  int64_t outer0 = in_size0, outer1 = in_size1;
  int64_t tile0 = in_size2, tile1 = in_size3;
  int64_t sl0 = in_stride0, sl1 = in_size2 * in_size3;
  int64_t sl2 = in_size3, sl3 = 1;
  if (flags & kTransposeOuter) {
    swap_i64(&outer0, &outer1);
    swap_i64(&sl0, &sl1);
  }
  if (flags & kTransposeInner) {
    swap_i64(&tile0, &tile1);
    swap_i64(&sl2, &sl3);
  }
  const char* in = (const char*)in_buffer;
  char* out = (char*)out_buffer;
  for (int64_t a0 = 0; a0 < outer0; ++a0)
    for (int64_t a1 = 0; a1 < outer1; ++a1)
      for (int64_t b0 = 0; b0 < tile0; ++b0)
        for (int64_t b1 = 0; b1 < tile1; ++b1) {
          const int64_t i0 = a0 * tile0 + b0, i1 = a1 * tile1 + b1;
          if (i0 >= out_size0 || i1 >= out_size1) continue;
          memcpy(out + (out_offset + i0 * out_stride0 + i1 * out_stride1) * es,
                 in + (in_offset + a0 * sl0 + a1 * sl1 + b0 * sl2 + b1 * sl3) * es,
                 es);
        }
  return 0;
}


/* conv_nchwc, f32 only (the reference has no other type):
 * input [N][IC_outer][IH][IW][c0], filter [OC_outer][IC_outer][FH][FW][c0][k0],
 * output [N][OC_outer][OH][OW][k0], strides in elements for the outer
 * dimensions as named; IW and FW steps are c0 and c0*k0. Accumulation order
 * (ic_outer, fh, fw, ci) per output element as in
 * conv_nchwc_tile_generic.c:34-57. Returns non-zero for an unknown type. */
UK_ORACLE_EXPORT int uk_oracle_conv_nchwc(
    const void* input_buffer, int64_t input_offset, int64_t input_stride_n,
    int64_t input_stride_ic_outer, int64_t input_stride_h, const void* filter_buffer,
    int64_t filter_offset, int64_t filter_stride_oc_outer, int64_t filter_stride_ic_outer,
    int64_t filter_stride_fh, void* output_buffer, int64_t output_offset,
    int64_t output_stride_n, int64_t output_stride_oc_outer, int64_t output_stride_oh,
    int64_t N, int64_t OC_outer, int64_t OH, int64_t OW, int64_t IC_outer, int64_t FH,
    int64_t FW, int32_t k0, int32_t c0, int32_t stride_h, int32_t stride_w, uint32_t flags,
    const uint64_t* cpu_data) {
  (void)cpu_data;
  if ((flags & kTypeMask) != 0x01) return 1; /* exported_bits.h:113-116 */
  const int accumulate = (flags & 0x100) != 0; /* exported_bits.h:119 */
  /* conv_nchwc.c:42-53 */
  if (N == 0 || OC_outer == 0 || OH == 0 || OW == 0) return 0;
  if ((IC_outer == 0 || FH == 0 || FW == 0) && accumulate) return 0;
  const float* in = (const float*)input_buffer + input_offset;
  const float* f = (const float*)filter_buffer + filter_offset;
  float* out = (float*)output_buffer + output_offset;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t oc = 0; oc < OC_outer; ++oc)
      for (int64_t oh = 0; oh < OH; ++oh)
        for (int64_t ow = 0; ow < OW; ++ow)
          for (int32_t ko = 0; ko < k0; ++ko) {
            float* o = out + n * output_stride_n + oc * output_stride_oc_outer +
                       oh * output_stride_oh + ow * k0 + ko;
            float acc = accumulate ? *o : 0.f;
            for (int64_t ic = 0; ic < IC_outer; ++ic)
              for (int64_t fh = 0; fh < FH; ++fh)
                for (int64_t fw = 0; fw < FW; ++fw)
                  for (int32_t ci = 0; ci < c0; ++ci) {
                    const float iv = in[n * input_stride_n + ic * input_stride_ic_outer +
                                        (oh * stride_h + fh) * input_stride_h +
                                        (ow * stride_w + fw) * c0 + ci];
                    const float fv = f[oc * filter_stride_oc_outer + ic * filter_stride_ic_outer +
                                       fh * filter_stride_fh + fw * (int64_t)c0 * k0 +
                                       (int64_t)ci * k0 + ko];
                    acc += iv * fv;
                  }
            *o = acc;
          }
  return 0;
}
