/*
 * Host layer of the MI355X ukernels: the C entry points of iree_uk_amd.h.
 *
 * Each entry point mirrors its CPU counterpart's control flow
 *   validate -> early return -> select kernel -> run
 * (runtime/src/iree/builtins/ukernel/mmt4d.c:116-142, pack.c:315-323,
 * unpack.c:249-257), with "run" being a HIP launch on the calling thread's
 * stream. Operands that live in ordinary host memory are staged through
 * device memory around the launch so that a caller written for the CPU
 * ukernels keeps working unchanged; device operands are used in place.
 *
 * Plain C: HIP is reached only through uk_hip_abi.h.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "uk_hip_abi.h"

/*---------------------------------------------------------------------------
 * Per-thread state. The entry points are re-entrant and may be called from
 * many host threads at once (runtime/src/iree/builtins/ukernel/README.md:26).
 *-------------------------------------------------------------------------*/

static _Thread_local void* tls_stream = 0;
static _Thread_local int tls_pointer_mode = IREE_UK_AMD_POINTER_MODE_AUTO;
static _Thread_local int tls_kernel_mode = IREE_UK_AMD_KERNEL_MODE_AUTO;
static _Thread_local int tls_status = 0;
static _Thread_local const char* tls_kernel_name = "";

static iree_uk_amd_assert_handler_t g_assert_handler = 0;

static void default_assert_handler(const char* file, int line,
                                   const char* function,
                                   const char* condition) {
  fflush(stdout);
  /* One fprintf call: may be reached from several threads at once. */
  fprintf(stderr, "%s:%d: %s: assertion failed: %s\n", file, line, function,
          condition);
  fflush(stderr);
  abort();
}

void iree_uk_amd_set_assert_handler(iree_uk_amd_assert_handler_t handler) {
  g_assert_handler = handler;
}

static void assert_fail(const char* file, int line, const char* function,
                        const char* condition) {
  iree_uk_amd_assert_handler_t h = g_assert_handler;
  tls_status = -1;
  (h ? h : default_assert_handler)(file, line, function, condition);
}

/* Checks a contract condition; on violation reports it through the hook and
 * makes the enclosing validate function return 0. */
#define UK_REQUIRE(cond)                                  \
  do {                                                    \
    if (!(cond)) {                                        \
      assert_fail(__FILE__, __LINE__, __func__, #cond);   \
      return 0;                                           \
    }                                                     \
  } while (0)

int iree_uk_amd_last_status(void) { return tls_status; }

const char* iree_uk_amd_last_status_string(void) {
  if (tls_status == 0) return "ok";
  if (tls_status == -1) return "contract violation";
  return iree_uk_amd_hip_error_string(tls_status);
}

void iree_uk_amd_set_stream(void* hip_stream) { tls_stream = hip_stream; }
void* iree_uk_amd_get_stream(void) { return tls_stream; }

int iree_uk_amd_synchronize(void) {
  return iree_uk_amd_hip_stream_synchronize(tls_stream);
}

void iree_uk_amd_set_pointer_mode(int mode) { tls_pointer_mode = mode; }
void iree_uk_amd_set_kernel_mode(int mode) { tls_kernel_mode = mode; }
const char* iree_uk_amd_last_kernel_name(void) { return tls_kernel_name; }
int iree_uk_amd_device_count(void) { return iree_uk_amd_hip_device_count(); }
const char* iree_uk_amd_version(void) { return "0.1"; }

/*---------------------------------------------------------------------------
 * Types.
 *-------------------------------------------------------------------------*/

typedef struct {
  int lhs_bits, rhs_bits, out_bits;
} mmt4d_bits_t;

/* Element widths of the (lhs, rhs, out) triple named by the flags' low byte
 * (mmt4d_internal.h:42-111). Returns 0 for an unknown type. */
static int mmt4d_type_bits(uint32_t flags, mmt4d_bits_t* b) {
  switch (flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: *b = (mmt4d_bits_t){32, 32, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *b = (mmt4d_bits_t){8, 8, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *b = (mmt4d_bits_t){16, 16, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16: *b = (mmt4d_bits_t){16, 16, 16}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *b = (mmt4d_bits_t){16, 16, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: *b = (mmt4d_bits_t){16, 16, 16}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: *b = (mmt4d_bits_t){16, 16, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: *b = (mmt4d_bits_t){16, 4, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: *b = (mmt4d_bits_t){16, 8, 32}; return 1;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: *b = (mmt4d_bits_t){8, 4, 32}; return 1;
    case IREE_UK_AMD_FLAG_MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: *b = (mmt4d_bits_t){8, 8, 32}; return 1;
    default: return 0;
  }
}

/* pack and unpack share type values; unpack has no 1-byte type
 * (exported_bits.h:56-62,73-79). */
static int pack_elem_bytes(uint32_t flags) {
  switch (flags & IREE_UK_FLAG_PACK_TYPE_MASK) {
    case IREE_UK_FLAG_PACK_TYPE_F32F32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_I8I8: return 1;
    case IREE_UK_FLAG_PACK_TYPE_I32I32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_F16F16: return 2;
    case IREE_UK_FLAG_PACK_TYPE_BF16BF16: return 2;
    default: return 0;
  }
}

static int unpack_elem_bytes(uint32_t flags) {
  if ((flags & IREE_UK_FLAG_UNPACK_TYPE_MASK) == IREE_UK_FLAG_PACK_TYPE_I8I8) {
    return 0;
  }
  return pack_elem_bytes(flags);
}

static int fits_unsigned_bits(int64_t v, int bits) {
  return v >= 0 && v < ((int64_t)1 << bits);
}

/* Smallest power of two >= x, for x >= 1. */
static int64_t ceil_pow2(int64_t x) {
  int64_t p = 1;
  while (p < x) p <<= 1;
  return p;
}

/*---------------------------------------------------------------------------
 * Staging of host operands.
 *
 * An operand is described as `rows` rows of `row_bytes` bytes, `pitch` bytes
 * apart (any sign, zero included), starting at `base`. A host operand gets a
 * device copy carved from the calling thread's staging arena (one grow-only
 * device allocation per thread, so a call allocates only when it needs more
 * than any call before it); the copies in and out are asynchronous and the
 * entry point synchronizes the stream once, before it returns.
 *   pitch >= row_bytes:   dense copy of the rows (device pitch = row_bytes);
 *   pitch <= -row_bytes:  the same, rows walked from the lowest address, and
 *                         the device pitch is -row_bytes;
 *   |pitch| < row_bytes:  rows overlap (broadcast for pitch 0): the byte range
 *                         they span is copied whole and the pitch is kept.
 * Only bytes that belong to a row are ever copied back, so bytes in the
 * stride gaps keep their host values and concurrent calls working on
 * neighbouring slabs do not overwrite each other.
 *-------------------------------------------------------------------------*/

typedef struct {
  char* host_base;   /* first byte the operand touches, in caller memory */
  int64_t pitch;     /* caller pitch, bytes */
  int64_t row_bytes; /* bytes per row that the op may touch */
  int64_t rows;
  void* device;         /* device address standing for host_base, or NULL when
                           the operand is used in place */
  int64_t device_pitch; /* pitch of the device copy, bytes */
  /* the 2-D copy that moves it: */
  char* copy_host;
  int64_t copy_pitch, copy_row_bytes, copy_rows, copy_device_offset, arena_bytes;
  char* copy_device;
} staged_t;

static staged_t staged(const void* base, int64_t pitch, int64_t row_bytes,
                       int64_t rows) {
  staged_t s;
  memset(&s, 0, sizeof s);
  s.host_base = (char*)base;
  s.pitch = pitch;
  s.row_bytes = row_bytes;
  s.rows = rows;
  return s;
}

static int is_device_pointer(const void* p, int* status) {
  if (tls_pointer_mode == IREE_UK_AMD_POINTER_MODE_DEVICE) return 1;
  int is_dev = 0;
  int st = iree_uk_amd_hip_classify_pointer(p, &is_dev);
  if (st) *status = st;
  return is_dev;
}

/* Decides how operand `s` travels; arena_bytes stays 0 for an operand that is
 * empty or already on the device. Returns 0 or a HIP status. */
static int stage_plan(staged_t* s) {
  s->device = 0;
  s->arena_bytes = 0;
  if (s->rows <= 0 || s->row_bytes <= 0) return 0;
  int st = 0;
  if (is_device_pointer(s->host_base, &st)) return st;
  if (st) return st;
  const int64_t last = (s->rows - 1) * s->pitch; /* offset of the last row */
  if (s->rows == 1 || s->pitch >= s->row_bytes) {
    s->copy_host = s->host_base;
    s->copy_pitch = s->rows == 1 ? s->row_bytes : s->pitch;
    s->copy_row_bytes = s->row_bytes;
    s->copy_rows = s->rows;
    s->copy_device_offset = 0;
    s->device_pitch = s->row_bytes;
  } else if (s->pitch <= -s->row_bytes) {
    s->copy_host = s->host_base + last;
    s->copy_pitch = -s->pitch;
    s->copy_row_bytes = s->row_bytes;
    s->copy_rows = s->rows;
    s->copy_device_offset = (s->rows - 1) * s->row_bytes;
    s->device_pitch = -s->row_bytes;
  } else {
    const int64_t lowest = last < 0 ? last : 0;
    s->copy_host = s->host_base + lowest;
    s->copy_row_bytes = (last < 0 ? -last : last) + s->row_bytes;
    s->copy_pitch = s->copy_row_bytes;
    s->copy_rows = 1;
    s->copy_device_offset = -lowest;
    s->device_pitch = s->pitch;
  }
  s->arena_bytes = (s->copy_row_bytes * s->copy_rows + 255) & ~(int64_t)255;
  return 0;
}

/* Gives every host operand of `ops` its device copy and starts the copies in
 * (`copy_in[i]` says whether the kernel needs operand i's current contents).
 * Returns 0 or a HIP status. */
static int stage_in(staged_t** ops, const int* copy_in, int count) {
  int64_t total = 0;
  for (int i = 0; i < count; ++i) {
    int st = stage_plan(ops[i]);
    if (st) return st;
    total += ops[i]->arena_bytes;
  }
  if (!total) return 0;
  void* arena = 0;
  int st = iree_uk_amd_hip_staging_reserve(&arena, total);
  if (st) return st;
  char* next = (char*)arena;
  for (int i = 0; i < count; ++i) {
    staged_t* s = ops[i];
    if (!s->arena_bytes) continue;
    s->copy_device = next;
    s->device = next + s->copy_device_offset;
    next += s->arena_bytes;
    if (!copy_in[i]) continue;
    st = iree_uk_amd_hip_copy2d_to_device(s->copy_device, s->copy_row_bytes,
                                          s->copy_host, s->copy_pitch,
                                          s->copy_row_bytes, s->copy_rows,
                                          tls_stream);
    if (st) return st;
  }
  return 0;
}

static int stage_out(staged_t* s) {
  if (!s->device) return 0;
  return iree_uk_amd_hip_copy2d_to_host(s->copy_host, s->copy_pitch,
                                        s->copy_device, s->copy_row_bytes,
                                        s->copy_row_bytes, s->copy_rows,
                                        tls_stream);
}

/* Ends a call that staged something: waits for the kernel and the copies, so
 * the caller's memory is final (and free to reuse) when the entry point
 * returns, and the arena is free for the thread's next call. */
static int stage_finish(int st, staged_t** ops, int count) {
  int any = 0;
  for (int i = 0; i < count; ++i) any |= ops[i]->device != 0;
  if (any) {
    int st2 = iree_uk_amd_hip_stream_synchronize(tls_stream);
    if (!st) st = st2;
  }
  return st;
}

/*---------------------------------------------------------------------------
 * mmt4d
 *-------------------------------------------------------------------------*/

/* mmt4d.c:12-48, plus the f8 extension type. */
static int mmt4d_validate(const iree_uk_mmt4d_params_t* p) {
  const uint32_t allflags =
      IREE_UK_FLAG_MMT4D_TYPE_MASK | IREE_UK_FLAG_MMT4D_ACCUMULATE |
      IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS |
      IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  UK_REQUIRE(!(p->flags & ~allflags));
  mmt4d_bits_t bits;
  UK_REQUIRE(mmt4d_type_bits(p->flags, &bits));
  UK_REQUIRE(fits_unsigned_bits(p->M, 31));
  UK_REQUIRE(fits_unsigned_bits(p->N, 31));
  UK_REQUIRE(fits_unsigned_bits(p->K, 31));
  UK_REQUIRE(fits_unsigned_bits(p->M0, 15));
  UK_REQUIRE(fits_unsigned_bits(p->N0, 15));
  UK_REQUIRE(fits_unsigned_bits(p->K0, 15));
  UK_REQUIRE(bits.out_bits >= 8);
  UK_REQUIRE(!((p->K0 * bits.lhs_bits) % 8));
  UK_REQUIRE(!((p->K0 * bits.rhs_bits) % 8));
  UK_REQUIRE(!((p->lhs_stride0 * bits.lhs_bits) % 8));
  UK_REQUIRE(!((p->rhs_stride0 * bits.rhs_bits) % 8));
  /* Not asserted upstream but assumed by its pointer arithmetic
   * (mmt4d.c:70-83): offsets of sub-byte operands land on byte boundaries. */
  UK_REQUIRE(!((p->lhs_offset * bits.lhs_bits) % 8));
  UK_REQUIRE(!((p->rhs_offset * bits.rhs_bits) % 8));
  return 1;
}

uint32_t iree_uk_mmt4d_info_p(const iree_uk_mmt4d_params_t* params) {
  return iree_uk_amd_hip_mmt4d_has_mfma_kernel(params->M0, params->N0,
                                               params->K0, params->flags)
             ? IREE_UK_FLAG_MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
             : 0;
}

uint32_t iree_uk_mmt4d_info(int32_t M0, int32_t N0, int32_t K0, uint32_t flags,
                            const uint64_t* cpu_data) {
  iree_uk_mmt4d_params_t params;
  memset(&params, 0, sizeof params);
  params.M0 = M0;
  params.N0 = N0;
  params.K0 = K0;
  params.flags = flags;
  params.cpu_data = cpu_data;
  return iree_uk_mmt4d_info_p(&params);
}

/* Runs a validated call. `rowmajor` NULL: the tiled result of iree_uk_mmt4d;
 * otherwise the result goes to the row-major matrix it describes (at
 * out_buffer + out_offset) and params->out_stride0 is not used. */
static void mmt4d_run(const iree_uk_mmt4d_params_t* params,
                      const iree_uk_amd_rowmajor_out_t* rowmajor) {
  /* mmt4d.c:126-139: without the fallback flag only an architecture-specific
   * (here: MFMA) kernel may serve the call. */
  if (!(params->flags &
        IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION) &&
      !iree_uk_mmt4d_info_p(params)) {
    assert_fail(__FILE__, __LINE__, __func__,
                "no target-specific tile function, and fallback not enabled.");
    return;
  }
  mmt4d_bits_t bits;
  mmt4d_type_bits(params->flags, &bits);
  iree_uk_mmt4d_params_t p = *params;
  iree_uk_amd_rowmajor_out_t rm;
  if (rowmajor) rm = *rowmajor;
  else memset(&rm, 0, sizeof rm);
  const int out_bytes = bits.out_bits / 8;
  staged_t lhs = staged((char*)p.lhs_buffer + p.lhs_offset * bits.lhs_bits / 8,
                  p.lhs_stride0 * bits.lhs_bits / 8,
                  p.K * p.M0 * p.K0 * bits.lhs_bits / 8, p.M);
  staged_t rhs = staged((char*)p.rhs_buffer + p.rhs_offset * bits.rhs_bits / 8,
                  p.rhs_stride0 * bits.rhs_bits / 8,
                  p.K * p.N0 * p.K0 * bits.rhs_bits / 8, p.N);
  staged_t out = staged((char*)p.out_buffer + p.out_offset * out_bytes,
                  p.out_stride0 * out_bytes, p.N * p.M0 * p.N0 * out_bytes,
                  p.M);
  if (rowmajor) {
    out.pitch = rm.stride0 * out_bytes;
    out.row_bytes = rm.size1 * out_bytes;
    out.rows = rm.size0;
  }
  /* Dequantizing store: the matrix is written in full and never read; the
   * initial accumulators (ACCUMULATE) come from a tiled buffer of their own. */
  const int dequant = rowmajor && rm.dequant;
  const int accumulate = (p.flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  staged_t acc = staged(0, 0, 0, 0), rscale = acc, cscale = acc;
  if (dequant) {
    if (accumulate) {
      acc.host_base = (char*)rm.acc;
      acc.pitch = rm.acc_stride0 * out_bytes;
      acc.row_bytes = p.N * p.M0 * p.N0 * out_bytes;
      acc.rows = p.M;
    }
    if (rm.row_scale) {
      rscale.host_base = (char*)rm.row_scale;
      rscale.pitch = rscale.row_bytes = rm.size0 * (int64_t)sizeof(float);
      rscale.rows = 1;
    }
    if (rm.col_scale) {
      cscale.host_base = (char*)rm.col_scale;
      cscale.pitch = cscale.row_bytes = rm.size1 * (int64_t)sizeof(float);
      cscale.rows = 1;
    }
  }
  staged_t* ops[6] = {&lhs, &rhs, &out, &acc, &rscale, &cscale};
  const int copy_in[6] = {1, 1, accumulate && !dequant, 1, 1, 1};
  int st = stage_in(ops, copy_in, 6);
  if (!st) {
    if (acc.device) {
      rm.acc = acc.device;
      rm.acc_stride0 = acc.device_pitch / out_bytes;
    }
    if (rscale.device) rm.row_scale = (const float*)rscale.device;
    if (cscale.device) rm.col_scale = (const float*)cscale.device;
    if (lhs.device) {
      p.lhs_buffer = lhs.device;
      p.lhs_offset = 0;
      p.lhs_stride0 = lhs.device_pitch * 8 / bits.lhs_bits;
    }
    if (rhs.device) {
      p.rhs_buffer = rhs.device;
      p.rhs_offset = 0;
      p.rhs_stride0 = rhs.device_pitch * 8 / bits.rhs_bits;
    }
    if (out.device) {
      p.out_buffer = out.device;
      p.out_offset = 0;
      p.out_stride0 = out.device_pitch / out_bytes;
      rm.stride0 = out.device_pitch / out_bytes;
    }
    st = iree_uk_amd_hip_launch_mmt4d(&p, rowmajor ? &rm : 0, tls_stream,
                                      tls_kernel_mode, &tls_kernel_name);
  }
  if (!st) st = stage_out(&out);
  st = stage_finish(st, ops, 6);
  tls_status = st;
}

void iree_uk_mmt4d_p(const iree_uk_mmt4d_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  if (!mmt4d_validate(params)) return;
  /* mmt4d.c:106-114 */
  if (params->M == 0 || params->N == 0 ||
      (params->K == 0 && (params->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE))) {
    return;
  }
  mmt4d_run(params, 0);
}

/* iree_uk_mmt4d_p without any allocation (see the header). */
void iree_uk_amd_mmt4d_no_alloc(const iree_uk_mmt4d_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  if (!mmt4d_validate(params)) return;
  /* mmt4d.c:106-114 */
  if (params->M == 0 || params->N == 0 ||
      (params->K == 0 && (params->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE))) {
    return;
  }
  /* A host operand would be staged through a device allocation: refuse it
   * before anything is launched. (K == 0 without ACCUMULATE reads no operand
   * but still writes the output.) */
  mmt4d_bits_t bits;
  mmt4d_type_bits(params->flags, &bits);
  const void* first_bytes[3] = {
      (const char*)params->lhs_buffer + params->lhs_offset * bits.lhs_bits / 8,
      (const char*)params->rhs_buffer + params->rhs_offset * bits.rhs_bits / 8,
      (const char*)params->out_buffer + params->out_offset * (bits.out_bits / 8)};
  for (int i = params->K == 0 ? 2 : 0; i < 3; ++i) {
    int st = 0;
    if (!is_device_pointer(first_bytes[i], &st)) {
      tls_status = st ? st : IREE_UK_AMD_STATUS_NEEDS_ALLOCATION;
      return;
    }
  }
  iree_uk_amd_hip_set_no_alloc(1);
  mmt4d_run(params, 0);
  iree_uk_amd_hip_set_no_alloc(0);
}

/* Fused mmt4d + unpack: validation is that of the two calls it stands for. */
static int mmt4d_unpack_validate(const iree_uk_amd_mmt4d_unpack_params_t* p,
                                 const iree_uk_mmt4d_params_t* mm) {
  if (!mmt4d_validate(mm)) return 0;
  UK_REQUIRE(p->out_size0 >= 0 && p->out_size0 <= p->M * p->M0);
  UK_REQUIRE(p->out_size1 >= 0 && p->out_size1 <= p->N * p->N0);
  return 1;
}

void iree_uk_amd_mmt4d_unpack_p(const iree_uk_amd_mmt4d_unpack_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  const iree_uk_mmt4d_params_t mm = {
      params->lhs_buffer, params->lhs_offset, params->lhs_stride0,
      params->rhs_buffer, params->rhs_offset, params->rhs_stride0,
      params->out_buffer, params->out_offset, /*out_stride0=*/0,
      params->M, params->N, params->K, params->M0, params->N0, params->K0,
      params->flags, params->cpu_data};
  if (!mmt4d_unpack_validate(params, &mm)) return;
  /* The early returns of the two calls (mmt4d.c:106-114, unpack.c:84-86). */
  if (params->M == 0 || params->N == 0 || params->out_size0 == 0 ||
      params->out_size1 == 0 ||
      (params->K == 0 && (params->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE))) {
    return;
  }
  iree_uk_amd_rowmajor_out_t rm;
  memset(&rm, 0, sizeof rm);
  rm.stride0 = params->out_stride0;
  rm.size0 = params->out_size0;
  rm.size1 = params->out_size1;
  mmt4d_run(&mm, &rm);
}

void iree_uk_amd_mmt4d_unpack(const void* lhs_buffer, iree_uk_index_t lhs_offset,
                              iree_uk_index_t lhs_stride0, const void* rhs_buffer,
                              iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0,
                              void* out_buffer, iree_uk_index_t out_offset,
                              iree_uk_index_t out_stride0, iree_uk_index_t out_size0,
                              iree_uk_index_t out_size1, iree_uk_index_t M,
                              iree_uk_index_t N, iree_uk_index_t K, int32_t M0,
                              int32_t N0, int32_t K0, uint32_t flags,
                              const uint64_t* cpu_data) {
  iree_uk_amd_mmt4d_unpack_params_t params = {
      lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0,
      out_buffer, out_offset, out_stride0, out_size0,  out_size1,  M,
      N,          K,          M0,          N0,         K0,         flags,
      cpu_data};
  iree_uk_amd_mmt4d_unpack_p(&params);
}

/* Fused mmt4d + dequantizing unpack: a 32-bit accumulator type, a matrix
 * inside the tiles, and an accumulator buffer whenever one is to be read. */
static int mmt4d_dequant_validate(
    const iree_uk_amd_mmt4d_dequant_unpack_params_t* p,
    const iree_uk_mmt4d_params_t* mm) {
  if (!mmt4d_validate(mm)) return 0;
  mmt4d_bits_t bits;
  mmt4d_type_bits(mm->flags, &bits);
  UK_REQUIRE(bits.out_bits == 32);
  UK_REQUIRE(p->out_size0 >= 0 && p->out_size0 <= p->M * p->M0);
  UK_REQUIRE(p->out_size1 >= 0 && p->out_size1 <= p->N * p->N0);
  UK_REQUIRE(!(p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) || p->acc_buffer != 0);
  return 1;
}

void iree_uk_amd_mmt4d_dequant_unpack_p(
    const iree_uk_amd_mmt4d_dequant_unpack_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  const iree_uk_mmt4d_params_t mm = {
      params->lhs_buffer, params->lhs_offset, params->lhs_stride0,
      params->rhs_buffer, params->rhs_offset, params->rhs_stride0,
      params->out_buffer, params->out_offset, /*out_stride0=*/0,
      params->M, params->N, params->K, params->M0, params->N0, params->K0,
      params->flags, params->cpu_data};
  if (!mmt4d_dequant_validate(params, &mm)) return;
  /* Nothing to write. Unlike iree_uk_mmt4d, K == 0 with ACCUMULATE is not a
   * no-op here: the accumulators still have to reach the matrix, scaled. */
  if (params->M == 0 || params->N == 0 || params->out_size0 == 0 ||
      params->out_size1 == 0) {
    return;
  }
  iree_uk_amd_rowmajor_out_t rm;
  memset(&rm, 0, sizeof rm);
  rm.stride0 = params->out_stride0;
  rm.size0 = params->out_size0;
  rm.size1 = params->out_size1;
  rm.dequant = 1;
  rm.row_scale = params->row_scale;
  rm.col_scale = params->col_scale;
  if (params->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) {
    rm.acc = (const char*)params->acc_buffer + params->acc_offset * 4;
    rm.acc_stride0 = params->acc_stride0;
  }
  mmt4d_run(&mm, &rm);
}

void iree_uk_amd_mmt4d_dequant_unpack(
    const void* lhs_buffer, iree_uk_index_t lhs_offset, iree_uk_index_t lhs_stride0,
    const void* rhs_buffer, iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0,
    const void* acc_buffer, iree_uk_index_t acc_offset, iree_uk_index_t acc_stride0,
    void* out_buffer, iree_uk_index_t out_offset, iree_uk_index_t out_stride0,
    iree_uk_index_t out_size0, iree_uk_index_t out_size1, const float* row_scale,
    const float* col_scale, iree_uk_index_t M, iree_uk_index_t N, iree_uk_index_t K,
    int32_t M0, int32_t N0, int32_t K0, uint32_t flags, const uint64_t* cpu_data) {
  iree_uk_amd_mmt4d_dequant_unpack_params_t params = {
      lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0,
      acc_buffer, acc_offset, acc_stride0, out_buffer, out_offset, out_stride0,
      out_size0,  out_size1,  row_scale,   col_scale,  M,          N,
      K,          M0,         N0,          K0,         flags,      cpu_data};
  iree_uk_amd_mmt4d_dequant_unpack_p(&params);
}

void iree_uk_mmt4d(const void* lhs_buffer, iree_uk_index_t lhs_offset,
                   iree_uk_index_t lhs_stride0, const void* rhs_buffer,
                   iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0,
                   void* out_buffer, iree_uk_index_t out_offset,
                   iree_uk_index_t out_stride0, iree_uk_index_t M,
                   iree_uk_index_t N, iree_uk_index_t K, int32_t M0,
                   int32_t N0, int32_t K0, uint32_t flags,
                   const uint64_t* cpu_data) {
  iree_uk_mmt4d_params_t params = {
      lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0,
      out_buffer, out_offset, out_stride0, M,          N,          K,
      M0,         N0,         K0,          flags,      cpu_data};
  iree_uk_mmt4d_p(&params);
}

/*---------------------------------------------------------------------------
 * pack
 *-------------------------------------------------------------------------*/

/* pack.c:51-104. The tile-size bound comes from the 4096-byte staging buffer
 * of the CPU implementation (pack.c:9,39-49); kept so that both accept the
 * same calls. */
static int pack_validate(const iree_uk_pack_params_t* p) {
  const uint32_t allflags = IREE_UK_FLAG_PACK_TRANSPOSE_INNER |
                            IREE_UK_FLAG_PACK_TRANSPOSE_OUTER |
                            IREE_UK_FLAG_PACK_TYPE_MASK;
  UK_REQUIRE(!(p->flags & ~allflags));
  const int es = pack_elem_bytes(p->flags);
  UK_REQUIRE(es != 0);
  UK_REQUIRE(p->in_size0 >= 0);
  UK_REQUIRE(p->in_size1 >= 0);
  UK_REQUIRE(p->out_size0 >= 0);
  UK_REQUIRE(p->out_size1 >= 0);
  UK_REQUIRE(p->out_size2 >= 0);
  UK_REQUIRE(p->out_size3 >= 0);
  UK_REQUIRE(p->in_stride0 >= 0);
  UK_REQUIRE(p->in_stride1 >= 0);
  UK_REQUIRE(p->out_stride0 >= 0);
  UK_REQUIRE(p->out_stride1 == p->out_size2 * p->out_size3);
  int64_t outer0 = p->out_size0, outer1 = p->out_size1;
  int64_t tile0 = p->out_size2, tile1 = p->out_size3;
  if (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER) {
    int64_t t = outer0; outer0 = outer1; outer1 = t;
  }
  if (p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER) {
    int64_t t = tile0; tile0 = tile1; tile1 = t;
  }
  UK_REQUIRE(outer0 * tile0 >= p->in_size0);
  UK_REQUIRE(outer1 * tile1 >= p->in_size1);
  UK_REQUIRE(tile0 * tile1 == 0 || ceil_pow2(tile0 * tile1 * es) <= 4096);
  return 1;
}

void iree_uk_pack_p(const iree_uk_pack_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  if (!pack_validate(params)) return;
  /* pack.c:106-109 */
  if (params->out_size0 == 0 || params->out_size1 == 0 ||
      params->out_size2 == 0 || params->out_size3 == 0) {
    return;
  }
  const int es = pack_elem_bytes(params->flags);
  iree_uk_pack_params_t p = *params;
  /* Source rows as the kernel may touch them: in_size1 elements in_stride1
   * apart. Gaps inside a row are copied along (reading them is harmless). */
  const int64_t in_row_elems =
      p.in_size1 > 0 ? (p.in_size1 - 1) * p.in_stride1 + 1 : 0;
  staged_t in = staged((char*)p.in_buffer + p.in_offset * es, p.in_stride0 * es,
                 in_row_elems * es, p.in_size0);
  staged_t out = staged((char*)p.out_buffer + p.out_offset * es, p.out_stride0 * es,
                  p.out_size1 * p.out_size2 * p.out_size3 * es, p.out_size0);
  staged_t* ops[2] = {&in, &out};
  const int copy_in[2] = {1, 0}; /* every byte of every tile is written */
  int st = stage_in(ops, copy_in, 2);
  if (!st) {
    if (in.device) {
      p.in_buffer = in.device;
      p.in_offset = 0;
      p.in_stride0 = in.device_pitch / es;
    }
    if (out.device) {
      p.out_buffer = out.device;
      p.out_offset = 0;
      p.out_stride0 = out.device_pitch / es;
    }
    st = iree_uk_amd_hip_launch_pack(&p, tls_stream, tls_kernel_mode,
                                     &tls_kernel_name);
  }
  if (!st) st = stage_out(&out);
  st = stage_finish(st, ops, 2);
  tls_status = st;
}

void iree_uk_pack(const void* in_buffer, iree_uk_index_t in_offset,
                  iree_uk_index_t in_stride0, iree_uk_index_t in_stride1,
                  void* out_buffer, iree_uk_index_t out_offset,
                  iree_uk_index_t out_stride0, iree_uk_index_t out_stride1,
                  iree_uk_index_t in_size0, iree_uk_index_t in_size1,
                  iree_uk_index_t out_size0, iree_uk_index_t out_size1,
                  iree_uk_index_t out_size2, iree_uk_index_t out_size3,
                  uint64_t padding_value, uint32_t flags,
                  const uint64_t* cpu_data) {
  iree_uk_pack_params_t params = {
      in_buffer, in_offset, in_stride0, in_stride1, out_buffer,    out_offset,
      out_stride0, out_stride1, in_size0, in_size1, out_size0,     out_size1,
      out_size2, out_size3, padding_value, flags,   cpu_data};
  iree_uk_pack_p(&params);
}

/*---------------------------------------------------------------------------
 * unpack
 *-------------------------------------------------------------------------*/

/* unpack.c:31-81. */
static int unpack_validate(const iree_uk_unpack_params_t* p) {
  const uint32_t allflags = IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER |
                            IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER |
                            IREE_UK_FLAG_UNPACK_TYPE_MASK;
  UK_REQUIRE(!(p->flags & ~allflags));
  const int es = unpack_elem_bytes(p->flags);
  UK_REQUIRE(es != 0);
  UK_REQUIRE(p->out_size0 >= 0);
  UK_REQUIRE(p->out_size1 >= 0);
  UK_REQUIRE(p->in_size0 >= 0);
  UK_REQUIRE(p->in_size1 >= 0);
  UK_REQUIRE(p->in_size2 >= 0);
  UK_REQUIRE(p->in_size3 >= 0);
  UK_REQUIRE(p->in_stride0 >= 0);
  UK_REQUIRE(p->in_stride1 == p->in_size2 * p->in_size3);
  UK_REQUIRE(p->out_stride0 >= 0);
  UK_REQUIRE(p->out_stride1 >= 0);
  int64_t outer0 = p->in_size0, outer1 = p->in_size1;
  int64_t tile0 = p->in_size2, tile1 = p->in_size3;
  if (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER) {
    int64_t t = outer0; outer0 = outer1; outer1 = t;
  }
  if (p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER) {
    int64_t t = tile0; tile0 = tile1; tile1 = t;
  }
  UK_REQUIRE(outer0 * tile0 >= p->out_size0);
  UK_REQUIRE(outer1 * tile1 >= p->out_size1);
  UK_REQUIRE(tile0 * tile1 == 0 || ceil_pow2(tile0 * tile1 * es) <= 4096);
  return 1;
}

void iree_uk_unpack_p(const iree_uk_unpack_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  if (!unpack_validate(params)) return;
  /* unpack.c:84-86 */
  if (params->out_size0 == 0 || params->out_size1 == 0) return;
  const int es = unpack_elem_bytes(params->flags);
  iree_uk_unpack_params_t p = *params;
  const int64_t out_row_elems = (p.out_size1 - 1) * p.out_stride1 + 1;
  staged_t in = staged((char*)p.in_buffer + p.in_offset * es, p.in_stride0 * es,
                 p.in_size1 * p.in_size2 * p.in_size3 * es, p.in_size0);
  staged_t out = staged((char*)p.out_buffer + p.out_offset * es, p.out_stride0 * es,
                  out_row_elems * es, p.out_size0);
  /* With a unit inner stride every byte of each destination row is written.
   * Otherwise the bytes between elements must survive the round trip, so the
   * rows are copied in first (and come back unchanged). */
  staged_t* ops[2] = {&in, &out};
  const int copy_in[2] = {1, p.out_stride1 != 1};
  int st = stage_in(ops, copy_in, 2);
  if (!st) {
    if (in.device) {
      p.in_buffer = in.device;
      p.in_offset = 0;
      p.in_stride0 = in.device_pitch / es;
    }
    if (out.device) {
      p.out_buffer = out.device;
      p.out_offset = 0;
      p.out_stride0 = out.device_pitch / es;
    }
    st = iree_uk_amd_hip_launch_unpack(&p, tls_stream, tls_kernel_mode,
                                       &tls_kernel_name);
  }
  if (!st) st = stage_out(&out);
  st = stage_finish(st, ops, 2);
  tls_status = st;
}

void iree_uk_unpack(const void* in_buffer, iree_uk_index_t in_offset,
                    iree_uk_index_t in_stride0, iree_uk_index_t in_stride1,
                    void* out_buffer, iree_uk_index_t out_offset,
                    iree_uk_index_t out_stride0, iree_uk_index_t out_stride1,
                    iree_uk_index_t in_size0, iree_uk_index_t in_size1,
                    iree_uk_index_t in_size2, iree_uk_index_t in_size3,
                    iree_uk_index_t out_size0, iree_uk_index_t out_size1,
                    uint32_t flags, const uint64_t* cpu_data) {
  iree_uk_unpack_params_t params = {
      in_buffer,   in_offset,   in_stride0, in_stride1, out_buffer, out_offset,
      out_stride0, out_stride1, in_size0,   in_size1,   in_size2,   in_size3,
      out_size0,   out_size1,   flags,      cpu_data};
  iree_uk_unpack_p(&params);
}

/*---------------------------------------------------------------------------
 * conv_nchwc
 *-------------------------------------------------------------------------*/

/* conv_nchwc.c:12-40 */
static int conv_nchwc_validate(const iree_uk_conv_nchwc_params_t* p) {
  const uint32_t allflags =
      IREE_UK_FLAG_CONV_NCHWC_TYPE_MASK | IREE_UK_FLAG_CONV_NCHWC_ACCUMULATE |
      IREE_UK_FLAG_CONV_NCHWC_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  UK_REQUIRE(!(p->flags & ~allflags));
  const uint32_t type_bits = p->flags & IREE_UK_FLAG_CONV_NCHWC_TYPE_MASK;
  UK_REQUIRE(type_bits > 0 && type_bits < IREE_UK_FLAG_CONV_NCHWC_TYPE_END);
  UK_REQUIRE(fits_unsigned_bits(p->N, 31));
  UK_REQUIRE(fits_unsigned_bits(p->OC_outer, 31));
  UK_REQUIRE(fits_unsigned_bits(p->OH, 31));
  UK_REQUIRE(fits_unsigned_bits(p->OW, 31));
  UK_REQUIRE(fits_unsigned_bits(p->IC_outer, 31));
  UK_REQUIRE(fits_unsigned_bits(p->FH, 31));
  UK_REQUIRE(fits_unsigned_bits(p->FW, 31));
  UK_REQUIRE(fits_unsigned_bits(p->k0, 15));
  UK_REQUIRE(fits_unsigned_bits(p->c0, 15));
  UK_REQUIRE(p->k0 > 0 && p->c0 > 0);
  UK_REQUIRE(p->stride_h > 0 && p->stride_w > 0);
  return 1;
}

/* conv_nchwc.c:200-218: the bit says that a tuned (here: MFMA) kernel serves
 * the tile shape, in which case the fallback flag is not needed. */
uint32_t iree_uk_conv_nchwc_info_p(const iree_uk_conv_nchwc_params_t* params) {
  return iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(params->k0, params->c0,
                                                    params->flags)
             ? IREE_UK_FLAG_CONV_NCHWC_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
             : 0;
}

uint32_t iree_uk_conv_nchwc_info(int32_t k0, int32_t c0, uint32_t flags,
                                 const uint64_t* cpu_data) {
  (void)cpu_data;
  return iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(k0, c0, flags)
             ? IREE_UK_FLAG_CONV_NCHWC_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
             : 0;
}

void iree_uk_conv_nchwc_p(const iree_uk_conv_nchwc_params_t* params) {
  tls_status = 0;
  tls_kernel_name = "";
  if (!conv_nchwc_validate(params)) return;
  /* conv_nchwc.c:42-53 */
  if (params->N == 0 || params->OC_outer == 0 || params->OH == 0 ||
      params->OW == 0) {
    return;
  }
  const int no_taps =
      params->IC_outer == 0 || params->FH == 0 || params->FW == 0;
  if (no_taps && (params->flags & IREE_UK_FLAG_CONV_NCHWC_ACCUMULATE)) return;
  /* conv_nchwc.c:139-152 */
  if (!iree_uk_conv_nchwc_info_p(params) &&
      !(params->flags &
        IREE_UK_FLAG_CONV_NCHWC_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)) {
    assert_fail(__FILE__, __LINE__, __func__,
                "no target-specific tile function, and fallback not enabled.");
    return;
  }
  iree_uk_conv_nchwc_params_t p = *params;
  /* Host operands are staged as the contiguous element range they span; the
   * output range travels to the device and back whole, so the elements
   * between its rows come back as they were. */
  const int64_t H = (p.OH - 1) * p.stride_h + p.FH;
  const int64_t W = (p.OW - 1) * p.stride_w + p.FW;
  const int64_t in_span =
      no_taps ? 0
              : (p.N - 1) * p.input_stride_n +
                    (p.IC_outer - 1) * p.input_stride_ic_outer +
                    (H - 1) * p.input_stride_h + W * p.c0;
  const int64_t f_span =
      no_taps ? 0
              : (p.OC_outer - 1) * p.filter_stride_oc_outer +
                    (p.IC_outer - 1) * p.filter_stride_ic_outer +
                    (p.FH - 1) * p.filter_stride_fh + p.FW * (int64_t)p.c0 * p.k0;
  const int64_t out_span = (p.N - 1) * p.output_stride_n +
                           (p.OC_outer - 1) * p.output_stride_oc_outer +
                           (p.OH - 1) * p.output_stride_oh + p.OW * (int64_t)p.k0;
  staged_t in = staged((char*)p.input_buffer + p.input_offset * 4, in_span * 4,
                 in_span * 4, in_span > 0 ? 1 : 0);
  staged_t flt = staged((char*)p.filter_buffer + p.filter_offset * 4, f_span * 4,
                  f_span * 4, f_span > 0 ? 1 : 0);
  staged_t out = staged((char*)p.output_buffer + p.output_offset * 4, out_span * 4,
                  out_span * 4, 1);
  staged_t* ops[3] = {&in, &flt, &out};
  const int copy_in[3] = {1, 1, 1};
  int st = stage_in(ops, copy_in, 3);
  if (!st) {
    if (in.device) { p.input_buffer = in.device; p.input_offset = 0; }
    if (flt.device) { p.filter_buffer = flt.device; p.filter_offset = 0; }
    if (out.device) { p.output_buffer = out.device; p.output_offset = 0; }
    st = iree_uk_amd_hip_launch_conv_nchwc(&p, tls_stream, tls_kernel_mode,
                                           &tls_kernel_name);
  }
  if (!st) st = stage_out(&out);
  st = stage_finish(st, ops, 3);
  tls_status = st;
}

void iree_uk_conv_nchwc(
    const void* input_buffer, iree_uk_index_t input_offset,
    iree_uk_index_t input_stride_n, iree_uk_index_t input_stride_ic_outer,
    iree_uk_index_t input_stride_h, const void* filter_buffer,
    iree_uk_index_t filter_offset, iree_uk_index_t filter_stride_oc_outer,
    iree_uk_index_t filter_stride_ic_outer, iree_uk_index_t filter_stride_fh,
    void* output_buffer, iree_uk_index_t output_offset,
    iree_uk_index_t output_stride_n, iree_uk_index_t output_stride_oc_outer,
    iree_uk_index_t output_stride_oh, iree_uk_index_t N,
    iree_uk_index_t OC_outer, iree_uk_index_t OH, iree_uk_index_t OW,
    iree_uk_index_t IC_outer, iree_uk_index_t FH, iree_uk_index_t FW,
    int32_t k0, int32_t c0, int32_t stride_h, int32_t stride_w, uint32_t flags,
    const uint64_t* cpu_data) {
  iree_uk_conv_nchwc_params_t params = {
      input_buffer, input_offset, input_stride_n, input_stride_ic_outer,
      input_stride_h, filter_buffer, filter_offset, filter_stride_oc_outer,
      filter_stride_ic_outer, filter_stride_fh, output_buffer, output_offset,
      output_stride_n, output_stride_oc_outer, output_stride_oh, N, OC_outer,
      OH, OW, IC_outer, FH, FW, k0, c0, stride_h, stride_w, flags,
      /*ow_count=*/0, cpu_data};
  iree_uk_conv_nchwc_p(&params);
}

/*---------------------------------------------------------------------------
 * query_tile_sizes
 *-------------------------------------------------------------------------*/

/* query_tile_sizes.c:43-75 with the gfx950 answer in place of a CPU one:
 * 16x16 output tiles (one MFMA 16x16 accumulator block) and a K0 that gives
 * each tile row 16..32 contiguous bytes, which the MFMA kernels can feed to
 * the matrix cores without regrouping bytes. */
void iree_uk_query_tile_sizes_2d(
    const iree_uk_query_tile_sizes_2d_params_t* params,
    iree_uk_query_tile_sizes_2d_out_params_t* out_params) {
  tls_status = 0;
  const uint32_t op =
      params->flags & IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK;
  const uint32_t role =
      params->flags & IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK;
  int M = 16, N = 16, K = 0;
  switch (op) {
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32: K = 4; break;
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32: K = 16; break;
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32:
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16:
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32:
    case IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16: K = 8; break;
    default:
      assert_fail(__FILE__, __LINE__, __func__, "operation is a known matmul");
      return;
  }
  if (role == IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS) {
    out_params->tile_size0 = M;
    out_params->tile_size1 = K;
  } else if (role == IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS) {
    out_params->tile_size0 = N;
    out_params->tile_size1 = K;
  } else if (role == IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT) {
    out_params->tile_size0 = M;
    out_params->tile_size1 = N;
  } else {
    assert_fail(__FILE__, __LINE__, __func__, "operand role is LHS, RHS or RESULT");
  }
}
