/*
 * Driver of the sanitizer build (`make -C oracle asan`): runs the product's
 * plain-C host layer (iree_amd/csrc/uk_host.c, uk_plugin.c) on the CPU, with
 * the stand-ins of asan_hip_stubs.c behind it, under AddressSanitizer + UBSan:
 *   - every entry point on host operands with loose strides and offsets: the
 *     staged result must equal the oracle called directly on the same bytes,
 *     over the whole buffer (stride gaps and slack included);
 *   - contract violations report through the assert hook and return;
 *   - the early-return cases (mmt4d.c:106-114, pack.c:106-109, unpack.c:84-86)
 *     touch no buffer (NULL pointers);
 *   - the executable-plugin face resolves its imports and its thunks run.
 * Exit status 0 = all of it held and no sanitizer report was raised.
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "iree_uk_amd.h"

int uk_oracle_mmt4d(const void*, int64_t, int64_t, const void*, int64_t, int64_t, void*, int64_t,
                    int64_t, int64_t, int64_t, int64_t, int32_t, int32_t, int32_t, uint32_t,
                    const uint64_t*);
int uk_oracle_pack(const void*, int64_t, int64_t, int64_t, void*, int64_t, int64_t, int64_t, int64_t,
                   int64_t, int64_t, int64_t, int64_t, int64_t, uint64_t, uint32_t, const uint64_t*);
int uk_oracle_unpack(const void*, int64_t, int64_t, int64_t, void*, int64_t, int64_t, int64_t,
                     int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, uint32_t,
                     const uint64_t*);
const void* iree_hal_executable_plugin_query(uint32_t max_version, void* reserved);
void asan_stubs_release(void); /* asan_hip_stubs.c: frees its stand-in for the staging arena */

static int failures = 0;
static int violations = 0;
#define CHECK(cond)                                                         \
  do {                                                                      \
    if (!(cond)) {                                                          \
      fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      ++failures;                                                           \
    }                                                                       \
  } while (0)

static void on_violation(const char* file, int line, const char* function, const char* condition) {
  (void)file; (void)line; (void)function; (void)condition;
  ++violations;
}

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) {
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  return (uint32_t)(rng_state >> 33);
}
/* Exactly `n` bytes, so that an access one byte past the end is caught. */
static uint8_t* random_bytes(size_t n, int small_values) {
  uint8_t* p = (uint8_t*)malloc(n ? n : 1);
  for (size_t i = 0; i < n; ++i) p[i] = (uint8_t)(small_values ? rnd() % 3 : rnd());
  return p;
}
static uint8_t* clone(const uint8_t* p, size_t n) {
  uint8_t* q = (uint8_t*)malloc(n ? n : 1);
  memcpy(q, p, n);
  return q;
}

static void mmt4d_case(uint32_t type, int lb, int rb, int ob, int M, int N, int K, int M0, int N0,
                       int K0, int accumulate, int slack) {
  const uint32_t flags = type | (accumulate ? IREE_UK_FLAG_MMT4D_ACCUMULATE : 0) |
                         IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  const int64_t ls = (int64_t)K * M0 * K0 + slack, rs = (int64_t)K * N0 * K0 + slack,
                os = (int64_t)N * M0 * N0 + slack, off = slack;
  const size_t lbytes = (size_t)((off + (int64_t)M * ls) * lb / 8),
               rbytes = (size_t)((off + (int64_t)N * rs) * rb / 8),
               obytes = (size_t)((off + (int64_t)M * os) * ob / 8);
  /* Small integers keep float products and sums exact in any order. */
  uint8_t* lhs = random_bytes(lbytes, lb == 32);
  uint8_t* rhs = random_bytes(rbytes, rb == 32);
  if (lb == 32) for (size_t i = 0; i + 4 <= lbytes; i += 4) { float v = (float)(lhs[i] % 3); memcpy(lhs + i, &v, 4); }
  if (rb == 32) for (size_t i = 0; i + 4 <= rbytes; i += 4) { float v = (float)(rhs[i] % 3); memcpy(rhs + i, &v, 4); }
  uint8_t* out_a = random_bytes(obytes, ob == 32 && lb == 32);
  if (lb == 32) for (size_t i = 0; i + 4 <= obytes; i += 4) { float v = (float)(out_a[i] % 3); memcpy(out_a + i, &v, 4); }
  uint8_t* out_b = clone(out_a, obytes);
  CHECK(uk_oracle_mmt4d(lhs, off, ls, rhs, off, rs, out_a, off, os, M, N, K, M0, N0, K0, flags, 0) == 0);
  iree_uk_mmt4d(lhs, off, ls, rhs, off, rs, out_b, off, os, M, N, K, M0, N0, K0, flags, 0);
  CHECK(iree_uk_amd_last_status() == 0);
  CHECK(memcmp(out_a, out_b, obytes) == 0);
  free(lhs); free(rhs); free(out_a); free(out_b);
}

/* Row pitches that a dense 2-D copy cannot express: `mode` 0 loose positive,
 * 1 negative (rows walked downwards in memory), 2 zero (every row the same
 * memory), 3 and 4 positive and negative pitches shorter than a row (rows
 * overlap). The buffer holds exactly the spanned range. */
static int64_t pitch_of(int mode, int64_t dense) {
  switch (mode) {
    case 1: return -(dense + 2);
    case 2: return 0;
    case 3: return dense / 2;
    case 4: return -(dense / 2);
    default: return dense + 2;
  }
}
static void mmt4d_pitch_case(uint32_t type, int lb, int rb, int ob, int lhs_mode, int rhs_mode,
                             int out_mode, int accumulate) {
  enum { M = 3, N = 2, K = 2, M0 = 4, N0 = 4, K0 = 2 };
  const uint32_t flags = type | (accumulate ? IREE_UK_FLAG_MMT4D_ACCUMULATE : 0) |
                         IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  const int64_t dl = K * M0 * K0, dr = K * N0 * K0, dout = N * M0 * N0;
  const int64_t ls = pitch_of(lhs_mode, dl), rs = pitch_of(rhs_mode, dr), os = pitch_of(out_mode, dout);
  const int64_t loff = ls < 0 ? -(M - 1) * ls : 0, roff = rs < 0 ? -(N - 1) * rs : 0,
                ooff = os < 0 ? -(M - 1) * os : 0;
  const size_t lbytes = (size_t)(((M - 1) * (ls < 0 ? -ls : ls) + dl) * lb / 8),
               rbytes = (size_t)(((N - 1) * (rs < 0 ? -rs : rs) + dr) * rb / 8),
               obytes = (size_t)(((M - 1) * (os < 0 ? -os : os) + dout) * ob / 8);
  uint8_t* lhs = random_bytes(lbytes, 0);
  uint8_t* rhs = random_bytes(rbytes, 0);
  uint8_t* out_a = random_bytes(obytes, 0);
  uint8_t* out_b = clone(out_a, obytes);
  CHECK(uk_oracle_mmt4d(lhs, loff, ls, rhs, roff, rs, out_a, ooff, os, M, N, K, M0, N0, K0, flags, 0) == 0);
  iree_uk_mmt4d(lhs, loff, ls, rhs, roff, rs, out_b, ooff, os, M, N, K, M0, N0, K0, flags, 0);
  CHECK(iree_uk_amd_last_status() == 0);
  CHECK(memcmp(out_a, out_b, obytes) == 0);
  free(lhs); free(rhs); free(out_a); free(out_b);
}

static void pack_unpack_case(uint32_t type, int es, int rows, int cols, int t0, int t1,
                             uint32_t transpose, int slack) {
  const int inner = (transpose & IREE_UK_FLAG_PACK_TRANSPOSE_INNER) != 0;
  const int outer = (transpose & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER) != 0;
  /* (t0, t1): tile extent along rows / columns of the 2-D matrix. */
  const int64_t o0 = (rows + t0 - 1) / t0, o1 = (cols + t1 - 1) / t1;
  const int64_t s0 = outer ? o1 : o0, s1 = outer ? o0 : o1;
  const int64_t s2 = inner ? t1 : t0, s3 = inner ? t0 : t1;
  const int64_t in_stride0 = cols + slack, out_stride1 = s2 * s3,
                out_stride0 = s1 * out_stride1 + slack, off = slack;
  const size_t in_bytes = (size_t)(off + (int64_t)rows * in_stride0) * es,
               out_bytes = (size_t)(off + s0 * out_stride0) * es;
  uint8_t* in = random_bytes(in_bytes, 0);
  uint8_t* pa = random_bytes(out_bytes, 0);
  uint8_t* pb = clone(pa, out_bytes);
  const uint64_t pad = 0x1122334455667788ull;
  CHECK(uk_oracle_pack(in, off, in_stride0, 1, pa, off, out_stride0, out_stride1, rows, cols, s0, s1,
                       s2, s3, pad, type | transpose, 0) == 0);
  iree_uk_pack(in, off, in_stride0, 1, pb, off, out_stride0, out_stride1, rows, cols, s0, s1, s2,
               s3, pad, type | transpose, 0);
  CHECK(iree_uk_amd_last_status() == 0);
  CHECK(memcmp(pa, pb, out_bytes) == 0);
  if (es != 1) { /* unpack has no 1-byte type (exported_bits.h:73-79) */
    uint8_t* ua = random_bytes(in_bytes, 0);
    uint8_t* ub = clone(ua, in_bytes);
    CHECK(uk_oracle_unpack(pa, off, out_stride0, out_stride1, ua, off, in_stride0, 1, s0, s1, s2, s3,
                           rows, cols, type | transpose, 0) == 0);
    iree_uk_unpack(pa, off, out_stride0, out_stride1, ub, off, in_stride0, 1, s0, s1, s2, s3, rows,
                   cols, type | transpose, 0);
    CHECK(iree_uk_amd_last_status() == 0);
    CHECK(memcmp(ua, ub, in_bytes) == 0);
    free(ua); free(ub);
  }
  free(in); free(pa); free(pb);
}

/* The part of the plugin ABI this driver needs
 * (runtime/src/iree/hal/local/executable_plugin.h:389-461). */
typedef struct { size_t count; const char* const* symbol_names; void** out_fn_ptrs; void** out_fn_contexts; } resolve_params_t;
typedef struct {
  const void* header;
  void* (*load)(const void* environment, size_t param_count, const void* params, void** out_self);
  void (*unload)(void* self);
  void* (*resolve)(void* self, const resolve_params_t* params, uint32_t* out_resolution);
} plugin_v0_t;
typedef int (*import_fn_t)(void* params_ptr, void* context, void* reserved);

static void plugin_checks(void) {
  CHECK(iree_hal_executable_plugin_query(0, 0) == 0);
  const plugin_v0_t* plugin = (const plugin_v0_t*)iree_hal_executable_plugin_query(1, 0);
  CHECK(plugin != 0);
  if (!plugin) return;
  void* self = (void*)1;
  const uint64_t env[2] = {0, 0};
  CHECK(((uintptr_t)plugin->load(env, 0, 0, &self) & 0x1F) == 0);
  const char* names[4] = {"iree_uk_mmt4d", "?no_such_symbol", "iree_uk_pack", "no_such_required"};
  void* fns[4] = {0, 0, 0, 0};
  void* ctxs[4] = {0, 0, 0, 0};
  resolve_params_t rp = {3, names, fns, ctxs};
  uint32_t resolution = 77;
  CHECK(((uintptr_t)plugin->resolve(self, &rp, &resolution) & 0x1F) == 0);
  CHECK(resolution == 1 && fns[0] && !fns[1] && fns[2]);
  rp.count = 4;
  CHECK(((uintptr_t)plugin->resolve(self, &rp, &resolution) & 0x1F) == 5);
  /* The mmt4d import: one dummy i32 result, then the params struct. */
  struct { int32_t unused_result; iree_uk_mmt4d_params_t p; } call;
  memset(&call, 0, sizeof call);
  int8_t lhs[2 * 4 * 8], rhs[3 * 4 * 8];
  int32_t got[2 * 3 * 4 * 4], want[2 * 3 * 4 * 4];
  for (size_t i = 0; i < sizeof lhs; ++i) lhs[i] = (int8_t)rnd();
  for (size_t i = 0; i < sizeof rhs; ++i) rhs[i] = (int8_t)rnd();
  memset(got, 0x55, sizeof got);
  memset(want, 0x55, sizeof want);
  call.p.lhs_buffer = lhs; call.p.lhs_stride0 = 32;
  call.p.rhs_buffer = rhs; call.p.rhs_stride0 = 32;
  call.p.out_buffer = got; call.p.out_stride0 = 48;
  call.p.M = 2; call.p.N = 3; call.p.K = 1; call.p.M0 = 4; call.p.N0 = 4; call.p.K0 = 8;
  call.p.flags = IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 | IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  CHECK(((import_fn_t)fns[0])(&call, 0, 0) == 0);
  CHECK(uk_oracle_mmt4d(lhs, 0, 32, rhs, 0, 32, want, 0, 48, 2, 3, 1, 4, 4, 8, call.p.flags, 0) == 0);
  CHECK(memcmp(got, want, sizeof got) == 0);
  plugin->unload(self);
}

int main(void) {
  iree_uk_amd_set_assert_handler(on_violation);
  /* mmt4d on staged host operands: every element width the staging code
   * distinguishes (4-bit rhs included), ragged tile shapes, loose strides. */
  for (int slack = 0; slack <= 2; slack += 2) {
    for (int acc = 0; acc <= 1; ++acc) {
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 8, 8, 32, 3, 2, 5, 16, 16, 2, acc, slack);
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 8, 8, 32, 1, 1, 1, 7, 3, 5, acc, slack);
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_F32F32F32, 32, 32, 32, 2, 3, 4, 8, 8, 1, acc, slack);
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_F16F16F32, 16, 16, 32, 2, 2, 3, 4, 6, 2, acc, slack);
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_S16S16S32, 16, 16, 32, 2, 2, 3, 4, 4, 2, acc, slack);
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_S8S4S32, 8, 4, 32, 2, 3, 2, 4, 8, 4, acc, slack);
      mmt4d_case(IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 8, 8, 32, 2, 2, 0, 4, 4, 2, acc, slack);
    }
  }
  CHECK(violations == 0);
  /* Negative, zero and overlapping row pitches on host operands; the output
   * with a negative pitch (overlapping output rows have no defined result). */
  for (int lm = 0; lm <= 4; ++lm) {
    for (int rm = 0; rm <= 4; ++rm) {
      for (int om = 0; om <= 1; ++om) {
        mmt4d_pitch_case(IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 8, 8, 32, lm, rm, om, (lm + rm) & 1);
        mmt4d_pitch_case(IREE_UK_FLAG_MMT4D_TYPE_S8S4S32, 8, 4, 32, lm, rm, om, rm & 1);
        mmt4d_pitch_case(IREE_UK_FLAG_MMT4D_TYPE_S16S16S32, 16, 16, 32, lm, rm, om, lm & 1);
      }
    }
  }
  CHECK(violations == 0);
  for (int slack = 0; slack <= 3; slack += 3) {
    for (uint32_t tr = 0; tr <= 0x300; tr += 0x100) {
      pack_unpack_case(IREE_UK_FLAG_PACK_TYPE_I8I8, 1, 7, 13, 4, 8, tr, slack);
      pack_unpack_case(IREE_UK_FLAG_PACK_TYPE_F32F32, 4, 33, 5, 16, 1, tr, slack);
      pack_unpack_case(IREE_UK_FLAG_PACK_TYPE_F16F16, 2, 16, 16, 16, 16, tr, slack);
      pack_unpack_case(IREE_UK_FLAG_PACK_TYPE_I32I32, 4, 1, 1, 8, 8, tr, slack);
    }
  }
  CHECK(violations == 0);
  /* Early returns: nothing may be dereferenced. */
  iree_uk_mmt4d(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 5, 5, 16, 16, 2,
                IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 | IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION, 0);
  iree_uk_mmt4d(0, 0, 0, 0, 0, 0, 0, 0, 0, 4, 4, 0, 16, 16, 2,
                IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 | IREE_UK_FLAG_MMT4D_ACCUMULATE |
                    IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION, 0);
  iree_uk_pack(0, 0, 0, 1, 0, 0, 0, 64, 0, 0, 0, 4, 8, 8, 0, IREE_UK_FLAG_PACK_TYPE_I8I8, 0);
  iree_uk_unpack(0, 0, 0, 64, 0, 0, 0, 1, 2, 2, 8, 8, 0, 7, IREE_UK_FLAG_UNPACK_TYPE_F32F32, 0);
  CHECK(violations == 0 && iree_uk_amd_last_status() == 0);
  /* Contract violations: reported, and the call returns without touching
   * anything (mmt4d.c:12-48, pack.c:51-104, unpack.c:31-82). */
  int before = violations;
  iree_uk_mmt4d(0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 16, 16, 2, 0x7F, 0);          /* unknown type */
  CHECK(violations == before + 1); before = violations;
  iree_uk_mmt4d(0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 16, 16, 2,
                IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 | 0x8000, 0);                       /* unknown flag */
  CHECK(violations == before + 1); before = violations;
  iree_uk_mmt4d(0, 0, 0, 0, 0, 0, 0, 0, 0, -1, 1, 1, 16, 16, 2,
                IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 0);                                /* negative size */
  CHECK(violations == before + 1); before = violations;
  { /* no matrix-core kernel (none here at all) and no fallback flag (mmt4d.c:126-139) */
    int8_t a[64] = {0}, b[64] = {0};
    int32_t c[16] = {0};
    iree_uk_mmt4d(a, 0, 16, b, 0, 16, c, 0, 16, 1, 1, 1, 4, 4, 4, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 0);
    CHECK(violations == before + 1); before = violations;
  }
  iree_uk_pack(0, 0, 8, 1, 0, 0, 64, 64, 8, 8, 1, 1, 8, 8, 0, 0x7F, 0);            /* unknown type */
  CHECK(violations == before + 1); before = violations;
  iree_uk_pack(0, 0, 8, 1, 0, 0, 64, 63, 8, 8, 1, 1, 8, 8, 0, IREE_UK_FLAG_PACK_TYPE_I8I8, 0); /* out_stride1 */
  CHECK(violations == before + 1); before = violations;
  iree_uk_unpack(0, 0, 64, 64, 0, 0, 8, 1, 1, 1, 8, 8, 8, 8, IREE_UK_FLAG_PACK_TYPE_I8I8, 0);  /* no 1-byte unpack */
  CHECK(violations == before + 1); before = violations;
  CHECK(iree_uk_mmt4d_info(16, 16, 2, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32, 0) == 0);
  plugin_checks();
  iree_uk_amd_set_assert_handler(0);
  asan_stubs_release();
  if (failures) {
    fprintf(stderr, "asan_host_driver: %d check(s) failed\n", failures);
    return 1;
  }
  printf("asan_host_driver: ok\n");
  return 0;
}
