/*
 * C-ABI of the MI355X (gfx950) data-tiled matmul ukernels: pack, mmt4d, unpack.
 *
 * The three entry points keep the argument lists, params structs, flag values,
 * type enums and tile-size conventions of the IREE CPU ukernels so that a
 * caller written against
 *   runtime/src/iree/builtins/ukernel/{mmt4d.h,pack.h,unpack.h,exported_bits.h}
 * links against this library unchanged.  Offsets and strides are counted in
 * elements, M/N/K of mmt4d are tile counts, and only the outermost stride of
 * each 4-D operand is free (inner dims are dense).
 *
 * What differs from the CPU ukernels:
 *   - the work runs as HIP kernels on the current HIP device;
 *   - buffers may be device memory (zero-copy, stream-ordered: the call
 *     returns once the kernels are enqueued on the calling thread's stream,
 *     see iree_uk_amd_set_stream / iree_uk_amd_synchronize) or host memory
 *     (staged through the GPU; the call returns when the result is in the
 *     host buffer);
 *   - `cpu_data` is accepted and ignored (NULL is allowed);
 *   - one mmt4d type value is added for f8E4M3FN x f8E4M3FN -> f32.
 *
 * Plain C; no HIP or torch types appear in any signature.
 */
#ifndef IREE_UK_AMD_H_
#define IREE_UK_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IREE_UK_AMD_EXPORT __attribute__((visibility("default")))

/* iree_uk_index_t is int64 on 64-bit targets (common.h:269-275). */
typedef int64_t iree_uk_index_t;

/*===--------------------------------------------------------------------===*/
/* Flag values (exported_bits.h:29-83). These are shared with the compiler   */
/* and therefore frozen.                                                     */
/*===--------------------------------------------------------------------===*/

/* mmt4d type enum, low byte of flags (exported_bits.h:29-41). */
enum {
  IREE_UK_FLAG_MMT4D_TYPE_MASK = 0xFF,
  IREE_UK_FLAG_MMT4D_TYPE_NONE = 0x00,
  IREE_UK_FLAG_MMT4D_TYPE_F32F32F32 = 0x01,
  IREE_UK_FLAG_MMT4D_TYPE_S8S8S32 = 0x02,
  IREE_UK_FLAG_MMT4D_TYPE_F16F16F32 = 0x03,
  IREE_UK_FLAG_MMT4D_TYPE_F16F16F16 = 0x04,
  IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32 = 0x05,
  IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16 = 0x06,
  IREE_UK_FLAG_MMT4D_TYPE_S16S16S32 = 0x07,
  IREE_UK_FLAG_MMT4D_TYPE_S16U4S32 = 0x08,
  IREE_UK_FLAG_MMT4D_TYPE_S16S8S32 = 0x09,
  IREE_UK_FLAG_MMT4D_TYPE_S8S4S32 = 0x0A,
  IREE_UK_FLAG_MMT4D_TYPE_END = 0x0B,
  /* The one deliberate addition: 8-bit float E4M3FN operands, f32 result.
   * Taken outside the contiguous upstream range so that a future upstream
   * 0x0B cannot collide. Element semantics follow
   * runtime/src/iree/base/internal/math.h:324-362,557-560 (no Inf, NaN is
   * S.1111.111, subnormals kept) and the f32-accumulating reference loop in
   * tools/testing/e2e/iree-e2e-matmul-test.cc:123-142. */
  IREE_UK_AMD_FLAG_MMT4D_TYPE_F8E4M3FNF8E4M3FNF32 = 0x80,
};

/* Subnormal f16 / bf16 operands. The reference's generic tile functions read
 * f16 and bf16 through a software conversion that turns subnormal inputs into
 * zero (common.h:664-700); its AVX-512 f16 tile function converts with
 * vcvtph2ps, which keeps them. Here the scalar kernel (GENERIC kernel mode,
 * and every call no matrix-core kernel serves) flushes them as the generic
 * tile functions do, bit for bit, and the matrix-core kernels keep them at
 * their value, as the instruction does. The two therefore differ on inputs
 * that hold subnormals, by at most the products of the flushed elements. */

/* mmt4d bit flags (exported_bits.h:44-46). */
enum {
  IREE_UK_FLAG_MMT4D_ACCUMULATE = 0x100,
  IREE_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION = 0x200,
  IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS = 0x400,
};

/* iree_uk_mmt4d_info result bits (exported_bits.h:49). On this target the bit
 * means "an MFMA kernel (not the scalar fallback kernel) serves this case".
 * It is not set for the 16-bit integer LHS types (S16S16S32, S16U4S32,
 * S16S8S32): the hardware has no 16-bit integer matrix instruction, and no
 * kernel serves every shape of a tile. With the fallback flag, S16S16S32
 * runs on the matrix cores as four 8-bit products per element pair (exact
 * modulo 2^32) when K is a whole number of 64-element steps and the result has
 * more than 32 rows and columns; otherwise, with K0 a power of two >= 2, these
 * types run on a vector dot-product kernel (v_dot2_i32_i16 fed from LDS,
 * bit-exact), about twenty times the scalar kernel's rate; other K0 on the
 * scalar kernel. */
enum {
  IREE_UK_FLAG_MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION = 0x1,
};

/* pack type enum and bit flags (exported_bits.h:56-66). */
enum {
  IREE_UK_FLAG_PACK_TYPE_MASK = 0xFF,
  IREE_UK_FLAG_PACK_TYPE_NONE = 0x00,
  IREE_UK_FLAG_PACK_TYPE_F32F32 = 0x01,
  IREE_UK_FLAG_PACK_TYPE_I8I8 = 0x02,
  IREE_UK_FLAG_PACK_TYPE_I32I32 = 0x03,
  IREE_UK_FLAG_PACK_TYPE_F16F16 = 0x04,
  IREE_UK_FLAG_PACK_TYPE_BF16BF16 = 0x05,
  IREE_UK_FLAG_PACK_TRANSPOSE_INNER = 0x100,
  IREE_UK_FLAG_PACK_TRANSPOSE_OUTER = 0x200,
};

/* unpack type enum and bit flags (exported_bits.h:73-83). There is no 1-byte
 * unpack type upstream (0x02 is reserved). */
enum {
  IREE_UK_FLAG_UNPACK_TYPE_MASK = 0xFF,
  IREE_UK_FLAG_UNPACK_TYPE_NONE = 0x00,
  IREE_UK_FLAG_UNPACK_TYPE_F32F32 = 0x01,
  IREE_UK_FLAG_UNPACK_TYPE_I32I32 = 0x03,
  IREE_UK_FLAG_UNPACK_TYPE_F16F16 = 0x04,
  IREE_UK_FLAG_UNPACK_TYPE_BF16BF16 = 0x05,
  IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER = 0x100,
  IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER = 0x200,
};

/* query_tile_sizes flags (exported_bits.h:91-107). */
enum {
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK = 0xFF,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS = 0x01,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS = 0x02,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT = 0x03,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK = 0xFF00,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32 = 0x0100,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32 = 0x0200,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32 = 0x0300,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16 = 0x0400,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32 = 0x0500,
  IREE_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16 = 0x0600,
};

/*===--------------------------------------------------------------------===*/
/* Params structs. Field order equals the entry-point argument order.        */
/*===--------------------------------------------------------------------===*/

/* Replaces iree_uk_mmt4d_params_t (mmt4d_internal.h:14-32). */
typedef struct iree_uk_mmt4d_params_t {
  const void* lhs_buffer; /* [M][K][M0][K0], outer stride lhs_stride0 */
  iree_uk_index_t lhs_offset;
  iree_uk_index_t lhs_stride0;
  const void* rhs_buffer; /* [N][K][N0][K0], outer stride rhs_stride0 */
  iree_uk_index_t rhs_offset;
  iree_uk_index_t rhs_stride0;
  void* out_buffer; /* [M][N][M0][N0], outer stride out_stride0 */
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t M;
  iree_uk_index_t N;
  iree_uk_index_t K;
  int32_t M0;
  int32_t N0;
  int32_t K0;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_mmt4d_params_t;

/* Replaces iree_uk_pack_params_t (pack_internal.h:12-30). */
typedef struct iree_uk_pack_params_t {
  const void* in_buffer; /* 2-D, strides in_stride0 / in_stride1 */
  iree_uk_index_t in_offset;
  iree_uk_index_t in_stride0;
  iree_uk_index_t in_stride1;
  void* out_buffer; /* 4-D [out_size0][out_size1][out_size2][out_size3] */
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t out_stride1; /* must equal out_size2*out_size3 (pack.c:72) */
  iree_uk_index_t in_size0;
  iree_uk_index_t in_size1;
  iree_uk_index_t out_size0;
  iree_uk_index_t out_size1;
  iree_uk_index_t out_size2;
  iree_uk_index_t out_size3;
  uint64_t padding_value; /* low elem_size bytes are used (pack.h:16-25) */
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_pack_params_t;

/* Replaces iree_uk_unpack_params_t (unpack_internal.h:12-29). */
typedef struct iree_uk_unpack_params_t {
  const void* in_buffer; /* 4-D [in_size0][in_size1][in_size2][in_size3] */
  iree_uk_index_t in_offset;
  iree_uk_index_t in_stride0;
  iree_uk_index_t in_stride1; /* must equal in_size2*in_size3 (unpack.c:49) */
  void* out_buffer; /* 2-D, strides out_stride0 / out_stride1 */
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t out_stride1;
  iree_uk_index_t in_size0;
  iree_uk_index_t in_size1;
  iree_uk_index_t in_size2;
  iree_uk_index_t in_size3;
  iree_uk_index_t out_size0;
  iree_uk_index_t out_size1;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_unpack_params_t;

/* Replaces iree_uk_query_tile_sizes_2d_params_t / _out_params_t
 * (query_tile_sizes.h:16-26). */
typedef struct iree_uk_query_tile_sizes_2d_params_t {
  uint32_t flags;
  iree_uk_index_t size0;
  iree_uk_index_t size1;
  const uint64_t* cpu_data;
} iree_uk_query_tile_sizes_2d_params_t;

typedef struct iree_uk_query_tile_sizes_2d_out_params_t {
  iree_uk_index_t tile_size0;
  iree_uk_index_t tile_size1;
} iree_uk_query_tile_sizes_2d_out_params_t;

/*===--------------------------------------------------------------------===*/
/* Entry points.                                                             */
/*===--------------------------------------------------------------------===*/

/* Replaces iree_uk_mmt4d (mmt4d.h:14-21, mmt4d.c:152-178).
 * For every i<M, j<N, i0<M0, j0<N0:
 *   OUT[i][j][i0][j0] = (ACCUMULATE ? OUT[i][j][i0][j0] : 0)
 *                     + sum_{k<K} sum_{k0<K0} LHS[i][k][i0][k0]*RHS[j][k][j0][k0]
 * Returns without touching OUT when M==0, N==0, or K==0 with ACCUMULATE
 * (mmt4d.c:106-114). Bytes of OUT outside the M0xN0 tiles are never written. */
IREE_UK_AMD_EXPORT void iree_uk_mmt4d(
    const void* lhs_buffer, iree_uk_index_t lhs_offset,
    iree_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0, void* out_buffer,
    iree_uk_index_t out_offset, iree_uk_index_t out_stride0, iree_uk_index_t M,
    iree_uk_index_t N, iree_uk_index_t K, int32_t M0, int32_t N0, int32_t K0,
    uint32_t flags, const uint64_t* cpu_data);

/* Replaces iree_uk_mmt4d_p (mmt4d_internal.h:35, mmt4d.c:116-142). */
IREE_UK_AMD_EXPORT void iree_uk_mmt4d_p(const iree_uk_mmt4d_params_t* params);

/* Replaces iree_uk_mmt4d_info (mmt4d.h:25-27, mmt4d.c:180-186) and
 * iree_uk_mmt4d_info_p (mmt4d_internal.h:40, mmt4d.c:144-150). */
IREE_UK_AMD_EXPORT uint32_t iree_uk_mmt4d_info(int32_t M0, int32_t N0,
                                               int32_t K0, uint32_t flags,
                                               const uint64_t* cpu_data);
IREE_UK_AMD_EXPORT uint32_t
iree_uk_mmt4d_info_p(const iree_uk_mmt4d_params_t* params);

/* Replaces iree_uk_pack (pack.h:26-34, pack.c:325-352). Writes every element
 * of every output tile, using the low elem_size bytes of padding_value where
 * the source index falls outside in_size0 x in_size1. */
IREE_UK_AMD_EXPORT void iree_uk_pack(
    const void* in_buffer, iree_uk_index_t in_offset,
    iree_uk_index_t in_stride0, iree_uk_index_t in_stride1, void* out_buffer,
    iree_uk_index_t out_offset, iree_uk_index_t out_stride0,
    iree_uk_index_t out_stride1, iree_uk_index_t in_size0,
    iree_uk_index_t in_size1, iree_uk_index_t out_size0,
    iree_uk_index_t out_size1, iree_uk_index_t out_size2,
    iree_uk_index_t out_size3, uint64_t padding_value, uint32_t flags,
    const uint64_t* cpu_data);

/* Replaces iree_uk_pack_p (pack_internal.h:32, pack.c:315-323). */
IREE_UK_AMD_EXPORT void iree_uk_pack_p(const iree_uk_pack_params_t* params);

/* Replaces iree_uk_unpack (unpack.h:17-25, unpack.c:259-285). Writes only
 * elements inside out_size0 x out_size1. */
IREE_UK_AMD_EXPORT void iree_uk_unpack(
    const void* in_buffer, iree_uk_index_t in_offset,
    iree_uk_index_t in_stride0, iree_uk_index_t in_stride1, void* out_buffer,
    iree_uk_index_t out_offset, iree_uk_index_t out_stride0,
    iree_uk_index_t out_stride1, iree_uk_index_t in_size0,
    iree_uk_index_t in_size1, iree_uk_index_t in_size2,
    iree_uk_index_t in_size3, iree_uk_index_t out_size0,
    iree_uk_index_t out_size1, uint32_t flags, const uint64_t* cpu_data);

/* Replaces iree_uk_unpack_p (unpack_internal.h:31, unpack.c:249-257). */
IREE_UK_AMD_EXPORT void iree_uk_unpack_p(const iree_uk_unpack_params_t* params);

/* Replaces iree_uk_query_tile_sizes_2d (query_tile_sizes.h:28-30,
 * query_tile_sizes.c:65-75): returns the (M0,K0) / (N0,K0) / (M0,N0) tile for
 * the operand role and matmul type in `flags`, chosen for the gfx950 MFMA
 * kernels instead of a CPU ISA. */
IREE_UK_AMD_EXPORT void iree_uk_query_tile_sizes_2d(
    const iree_uk_query_tile_sizes_2d_params_t* params,
    iree_uk_query_tile_sizes_2d_out_params_t* out_params);

/*===--------------------------------------------------------------------===*/
/* Contract-violation hook.                                                  */
/*===--------------------------------------------------------------------===*/

/* Replaces the embedder-provided iree_uk_assert_fail (common.h:307-308).
 * The entry points return void; contract violations (unknown flags or types,
 * negative sizes, out_stride1 != out_size2*out_size3, ...) are reported
 * through this hook and the call then returns without doing any work.
 * The default handler prints "file:line: function: assertion failed: cond"
 * to stderr and aborts, like tools/util.c:21-31. */
typedef void (*iree_uk_amd_assert_handler_t)(const char* file, int line,
                                             const char* function,
                                             const char* condition);
IREE_UK_AMD_EXPORT void iree_uk_amd_set_assert_handler(
    iree_uk_amd_assert_handler_t handler); /* NULL restores the default */

/*===--------------------------------------------------------------------===*/
/* Device control: has no counterpart in the reference, whose ukernels run   */
/* synchronously on the calling CPU thread.                                  */
/*===--------------------------------------------------------------------===*/

/* Status of the most recent entry-point call on this thread: 0 = OK, else a
 * hipError_t value (launch or staging failure), -1 (contract violation) or
 * one of the values below. */
enum {
  /* Not returned by this version of the library (kept so that the values
   * stay what callers compiled against): a call of iree_uk_amd_mmt4d_no_alloc
   * whose K-split workspace would exceed the static scratch array runs without
   * the split instead. */
  IREE_UK_AMD_STATUS_SCRATCH_TOO_SMALL = 100001,
  /* iree_uk_amd_mmt4d_no_alloc: an operand is ordinary host memory, which
   * would have to be staged through a device allocation. */
  IREE_UK_AMD_STATUS_NEEDS_ALLOCATION = 100002,
};
IREE_UK_AMD_EXPORT int iree_uk_amd_last_status(void);
IREE_UK_AMD_EXPORT const char* iree_uk_amd_last_status_string(void);

/* Stream (a hipStream_t passed as void*) that this thread's calls enqueue on.
 * NULL (the default) is the null stream. */
IREE_UK_AMD_EXPORT void iree_uk_amd_set_stream(void* hip_stream);
IREE_UK_AMD_EXPORT void* iree_uk_amd_get_stream(void);

/* Blocks until this thread's stream has drained. Returns 0 or a hipError_t. */
IREE_UK_AMD_EXPORT int iree_uk_amd_synchronize(void);

/* How buffer pointers are classified, per thread.
 *   AUTO  : ask the HIP runtime about the first byte each operand touches;
 *           host memory is staged through the GPU.
 *   DEVICE: the caller promises device-accessible memory; no query is made
 *           (saves ~1 us per operand on small problems). */
enum {
  IREE_UK_AMD_POINTER_MODE_AUTO = 0,
  IREE_UK_AMD_POINTER_MODE_DEVICE = 1,
};
IREE_UK_AMD_EXPORT void iree_uk_amd_set_pointer_mode(int mode);

/* Kernel selection override for testing and benchmarking, per thread.
 *   AUTO    : fastest kernel that serves the case.
 *   GENERIC : always the scalar any-shape kernels.
 *   MFMA_VARIANT + v : mmt4d takes MFMA workgroup shape v where it can serve
 *             the call (1 = 256x256, 2 = 128x128, 3 = 64x64, 4 = the M-thin
 *             kernels, 5 = the M-thin kernel on the transposed problem,
 *             6 = the 64x64 K-split kernel, 7 = 256x128, 8 = 128x512,
 *             9 / 10 = the persistent kernel in the 128x512 / 256x256 shape,
 *             11 = 64x64 with the deep pipeline, 12..15 = the narrow-row
 *             kernels in the 256x256 / 128x512 / 128x128 / 64x64 shapes)
 *             instead of choosing by problem size; pack/unpack as AUTO. */
enum {
  IREE_UK_AMD_KERNEL_MODE_AUTO = 0,
  IREE_UK_AMD_KERNEL_MODE_GENERIC = 1,
  IREE_UK_AMD_KERNEL_MODE_MFMA_VARIANT = 16,
};
IREE_UK_AMD_EXPORT void iree_uk_amd_set_kernel_mode(int mode);

/* iree_uk_mmt4d_info's bit promises a matrix-core kernel for the tile shape at
 * every M, N, K, for operands at any element-aligned address, as long as
 * strides are non-negative and every operand spans less than 2 GiB from its
 * first panel. Outside those limits the call is still served, with the same
 * result, by the scalar kernel (64-bit indexing), about 100x slower; this
 * counts such calls of the calling thread since it started, so a caller (or a
 * test) can see the cliff. iree_uk_amd_last_kernel_name names the kernel of
 * the latest call. No counterpart in the reference, whose tile functions take
 * any stride. */
IREE_UK_AMD_EXPORT uint64_t iree_uk_amd_mfma_decline_count(void);

/* iree_uk_mmt4d_p for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference. Same parameters, same result (bit
 * for bit, floats included, whenever both entry points split K alike: they
 * take the same kernel), with two differences:
 *   - every operand must already be device-accessible memory; a host operand
 *     fails with IREE_UK_AMD_STATUS_NEEDS_ALLOCATION (iree_uk_mmt4d would
 *     stage it through a device allocation);
 *   - when the kernel splits K over workgroups (M-thin or N-thin problems of
 *     few output blocks and a long K: the decode step of a linear layer), the
 *     slices' partial accumulators and arrival counters live in a static
 *     device array of the library, iree_uk_amd_no_alloc_scratch_bytes() bytes
 *     (8 MiB of partials + 16384 counters) held by every GPU the library runs
 *     on, instead of a buffer iree_uk_mmt4d allocates on first need. A call
 *     whose split would need more runs without the split (one workgroup per
 *     output block over all of K, which needs no scratch memory): the same
 *     integers, and float sums in the unsplit order.
 * (iree_uk_mmt4d itself, called on a stream that is being captured into a HIP
 * graph, never hands that stream one of its own workspaces - the graph would
 * outlive it - and runs such a call without the split.)
 * The call allocates nothing: no hipMalloc / hipFree, no allocating library
 * routine. All calls on one GPU share that GPU's array; the kernels leave its
 * counters at zero and write partials before reading them, so consecutive
 * calls need no clearing, but calls that OVERLAP on one GPU (two streams, two
 * threads) race on it: serialize them. Results through the status functions
 * as for every entry point. */
IREE_UK_AMD_EXPORT void iree_uk_amd_mmt4d_no_alloc(const iree_uk_mmt4d_params_t* params);
IREE_UK_AMD_EXPORT int64_t iree_uk_amd_no_alloc_scratch_bytes(void);

/* Tuning / test knob of the calling thread: into how many slices the M-thin /
 * N-thin mmt4d kernels split K across workgroups (0, the default: chosen from
 * the number of output blocks and compute units; 1: never). The slice count
 * the latest call used is iree_uk_amd_last_k_slices (1 = no split). */
IREE_UK_AMD_EXPORT void iree_uk_amd_set_k_slices(int n);
IREE_UK_AMD_EXPORT int iree_uk_amd_last_k_slices(void);

/* A hint of the calling thread about where its weights are. 1: the wide
 * operand of the decode-shaped (M-thin / N-thin) mmt4d calls that follow is
 * read from HBM every time, as the layers of a model that evict each other
 * from the caches are; such operands of 16 MB and more are then loaded
 * non-temporally (58.7 MB of weights that no cache holds: 16.8 -> 15.4 us). 0,
 * the default: ordinary loads, which are the faster ones when the same
 * weights are used again while the 256 MB memory-side cache still holds
 * them (12.3 against 14.3 us). Results are the same either way. No
 * counterpart in the reference, whose callers have no such cache to manage. */
IREE_UK_AMD_EXPORT void iree_uk_amd_set_streamed_weights(int on);

/* Tuning / test knob of the calling thread: how many workgroups the
 * persistent mmt4d kernels launch (each walks its share of the output blocks
 * with one software pipeline running across block boundaries). 0, the
 * default, is one workgroup per compute unit. No counterpart in the
 * reference. */
IREE_UK_AMD_EXPORT void iree_uk_amd_set_persistent_workgroups(int n);

/* Name of the kernel variant the most recent call on this thread launched
 * ("" if it returned early). Static storage; never NULL. */
IREE_UK_AMD_EXPORT const char* iree_uk_amd_last_kernel_name(void);

/* Measured ceilings for benchmark reports (no counterpart in the reference,
 * whose tools/mmt4d_benchmark.c and tools/pack_benchmark.c print rates with
 * nothing beside them).
 *
 * iree_uk_amd_probe_mfma_peak: a loop of nothing but matrix-core instructions
 * of the element type in `type_flags` (S8S8S32, F16F16F32, BF16BF16F32,
 * F32F32F32 or the f8 extension), 8 waves per workgroup with the register
 * blocking of the mmt4d kernels, `workgroups` workgroups (0 = two per compute
 * unit), `iters` passes over a wave's 32 accumulator blocks. The lanes take
 * their register operands once from `operands` (`operand_bytes` of device
 * memory, a multiple of 16): all-zero and random bytes give different clocks
 * on a power-limited part. `sink`: device memory, one int per thread, never
 * written in practice. Runs on `stream` (a hipStream_t) and waits for it.
 * Returns 0 or a hipError_t value; *ops_per_second receives the rate.
 *
 * iree_uk_amd_probe_copy2d: `iters` plain copies of `rows` rows of `row_bytes`
 * bytes between two pitches (everything 4-byte aligned): the ceiling of a
 * pack / unpack that moves the same matrix between the same pitches.
 * *seconds_per_copy receives the average of the fastest of five ways of
 * writing the copy (1, 4 or 8 vectors in flight per lane, ordinary or
 * non-temporal stores, non-temporal loads as well with 8 in flight, and one
 * whose stores cover only whole 128-byte lines of the destination whatever
 * its pitch).
 * iree_uk_amd_probe_copy2d_variants: the same, and seconds_per_variant[0..4]
 * (when not NULL) receive the average of every variant, the whole-line one
 * last. */
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_mfma_peak(
    uint32_t type_flags, const void* operands, int64_t operand_bytes, int iters,
    int workgroups, void* sink, void* stream, double* ops_per_second);
/* The s8 MFMA-only loop, its MFMAs written as assembly, with exactly
 * `waves_per_simd` (1 or 2) waves on every SIMD (one workgroup per CU): what a
 * lone wave can feed the matrix pipe against what two can. Arguments as for
 * iree_uk_amd_probe_mfma_peak. */
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_mfma_peak_waves(
    const void* operands, int64_t operand_bytes, int iters, int waves_per_simd,
    void* sink, void* stream, double* ops_per_second);
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_copy2d(
    const void* src, int64_t src_pitch, void* dst, int64_t dst_pitch,
    int64_t row_bytes, int64_t rows, int iters, void* stream,
    double* seconds_per_copy);
/* iree_uk_amd_probe_ds_read_tr16: one wave executes ds_read_b64_tr_b16, every
 * lane at the 16-bit index `lane_index[lane]` (device memory, 64 ints,
 * multiples of 4 below `lds_values` <= 16384) of an LDS image whose 16-bit
 * values equal their own indices; `out` (device memory, 256 shorts) receives
 * each lane's four values. Waits for `stream`. The fragment reads of the
 * mmt4d kernels for 2-byte tile rows rest on this instruction's lane mapping;
 * the test suite pins it through this call. No counterpart in the reference. */
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_ds_read_tr16(
    const int* lane_index, short* out, int lds_values, void* stream);
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_copy2d_variants(
    const void* src, int64_t src_pitch, void* dst, int64_t dst_pitch,
    int64_t row_bytes, int64_t rows, int iters, void* stream,
    double* seconds_per_copy, double* seconds_per_variant);

/* Per-kernel device timing for the calling thread. Between begin and end,
 * every kernel an entry point launches carries its own start/stop event pair
 * (the events timestamp the kernel itself, as a profiler would). end waits for
 * the kernels, writes up to `capacity` durations in microseconds to
 * elapsed_us[] in launch order with the launching op in kinds[] (0 pack,
 * 1 unpack, 2 mmt4d; either array may be NULL), and returns the number of
 * kernels launched since begin. */
IREE_UK_AMD_EXPORT void iree_uk_amd_timing_begin(void);
IREE_UK_AMD_EXPORT int iree_uk_amd_timing_end(double* elapsed_us, int* kinds,
                                              int capacity);

/* Host operands (ordinary memory, see the top of this file) are staged
 * through a device arena owned by the calling thread: one allocation per
 * device that grows to the largest call's need and is then reused, so that a
 * caller that always passes host pointers (the HAL executable-plugin thunks)
 * allocates a handful of times in its life. staging_bytes reports what the
 * calling thread holds; release_staging frees it (0 or a hipError_t value; a
 * later host-operand call allocates again), and so does the thread's end. Any pitch is staged, negative and
 * zero (broadcast) included. No counterpart in the reference. */
IREE_UK_AMD_EXPORT int64_t iree_uk_amd_staging_bytes(void);
IREE_UK_AMD_EXPORT int iree_uk_amd_release_staging(void);

/* Device buffers that iree_uk_mmt4d and iree_uk_conv_nchwc keep per calling
 * thread and stream beyond a call: the workspace of the thin kernels' K split
 * over workgroups (a few megabytes) and the buffer for operands the library
 * prepares before the matrix-core kernels run (4-bit weights expanded to s8
 * from 512 rows on, the right-hand side of s16 x s8 / s16 x u4 widened to s16,
 * narrow tile rows regrouped along K: as large as the prepared operands, at
 * most 2 GiB), which also holds the partial sums of a convolution whose input
 * channels are split over workgroups (at most 64 MB).
 * workspace_bytes reports what the calling thread holds; release_workspaces
 * frees it after waiting for the device (0 or a hipError_t value; a later
 * call allocates again), and so does the thread's end. Calls through
 * iree_uk_amd_mmt4d_no_alloc and calls on a stream that is being captured use
 * none of them. No counterpart in the reference. */
IREE_UK_AMD_EXPORT int64_t iree_uk_amd_workspace_bytes(void);
IREE_UK_AMD_EXPORT int iree_uk_amd_release_workspaces(void);

/* Device allocations (hipMalloc calls) the library has made in this process so
 * far, over all threads: the staging arenas and the workspaces above. A caller, or a test, can see with it that a call
 * allocated nothing (iree_uk_amd_mmt4d_no_alloc never does). No counterpart
 * in the reference. */
IREE_UK_AMD_EXPORT int64_t iree_uk_amd_device_alloc_count(void);

/* Number of devices visible to HIP (0 when there is none or no driver). */
IREE_UK_AMD_EXPORT int iree_uk_amd_device_count(void);

/* Library version, "major.minor". */
IREE_UK_AMD_EXPORT const char* iree_uk_amd_version(void);

/*===----------------------------------------------------------------------===*/
/* conv_nchwc                                                                  */
/*===----------------------------------------------------------------------===*/

/* The convolution ukernel of the same reference library
 * (runtime/src/iree/builtins/ukernel/conv_nchwc.h:14-31), kept so that the
 * library stands in for all of iree/builtins/ukernel/api.h. Tile shapes
 * k0 = 16, c0 a multiple of 16 (the reference's own tuned shape is 16x16,
 * arch/x86_64/conv_nchwc_x86_64_avx512_base.c:17-28) run on the matrix cores
 * (v_mfma_f32_16x16x4_f32; sums in MFMA order, equal to the reference's to f32
 * rounding and exactly where the partial sums are exact); every other shape on
 * a scalar kernel (one thread per output element, the reference's generic
 * accumulation order, bit-identical to it).
 *
 * input [N][IC_outer][IH][IW][c0], filter [OC_outer][IC_outer][FH][FW][c0][k0],
 * output [N][OC_outer][OH][OW][k0]; the named strides are in elements.
 * Flag values: exported_bits.h:113-124. */
enum {
  IREE_UK_FLAG_CONV_NCHWC_TYPE_MASK = 0xFF,
  IREE_UK_FLAG_CONV_NCHWC_TYPE_NONE = 0x00,
  IREE_UK_FLAG_CONV_NCHWC_TYPE_F32F32F32 = 0x01,
  IREE_UK_FLAG_CONV_NCHWC_TYPE_END = 0x02,
  IREE_UK_FLAG_CONV_NCHWC_ACCUMULATE = 0x100,
  IREE_UK_FLAG_CONV_NCHWC_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION = 0x200,
  IREE_UK_FLAG_CONV_NCHWC_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION = 0x1,
};

/* Replaces iree_uk_conv_nchwc_params_t (conv_nchwc_internal.h:12-46); field
 * order is the reference's, `ow_count` (a per-tile value its driver loop sets)
 * included and ignored. */
typedef struct iree_uk_conv_nchwc_params_t {
  const void* input_buffer;
  iree_uk_index_t input_offset;
  iree_uk_index_t input_stride_n;
  iree_uk_index_t input_stride_ic_outer;
  iree_uk_index_t input_stride_h;
  const void* filter_buffer;
  iree_uk_index_t filter_offset;
  iree_uk_index_t filter_stride_oc_outer;
  iree_uk_index_t filter_stride_ic_outer;
  iree_uk_index_t filter_stride_fh;
  void* output_buffer;
  iree_uk_index_t output_offset;
  iree_uk_index_t output_stride_n;
  iree_uk_index_t output_stride_oc_outer;
  iree_uk_index_t output_stride_oh;
  iree_uk_index_t N;
  iree_uk_index_t OC_outer;
  iree_uk_index_t OH;
  iree_uk_index_t OW;
  iree_uk_index_t IC_outer;
  iree_uk_index_t FH;
  iree_uk_index_t FW;
  int32_t k0;
  int32_t c0;
  int32_t stride_h;
  int32_t stride_w;
  uint32_t flags;
  iree_uk_index_t ow_count;
  const uint64_t* cpu_data;
} iree_uk_conv_nchwc_params_t;

/* Replaces iree_uk_conv_nchwc (conv_nchwc.h:14-27, conv_nchwc.c:157-198). */
IREE_UK_AMD_EXPORT void iree_uk_conv_nchwc(
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
    const uint64_t* cpu_data);
/* Replaces iree_uk_conv_nchwc_p (conv_nchwc_internal.h:48, conv_nchwc.c:132-155). */
IREE_UK_AMD_EXPORT void iree_uk_conv_nchwc_p(const iree_uk_conv_nchwc_params_t* params);
/* Replace iree_uk_conv_nchwc_info (conv_nchwc.h:29-31, conv_nchwc.c:210-218) and
 * iree_uk_conv_nchwc_info_p (conv_nchwc.c:200-208):
 * HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION for k0 = 16 with c0 a multiple of
 * 16, else 0 and callers must pass ALLOW_GENERIC_FALLBACK_TILE_FUNCTION. */
IREE_UK_AMD_EXPORT uint32_t iree_uk_conv_nchwc_info(int32_t k0, int32_t c0, uint32_t flags,
                                                    const uint64_t* cpu_data);
IREE_UK_AMD_EXPORT uint32_t iree_uk_conv_nchwc_info_p(
    const iree_uk_conv_nchwc_params_t* params);

/*===----------------------------------------------------------------------===*/
/* Fused mmt4d + unpack                                                        */
/*===----------------------------------------------------------------------===*/

/* No counterpart in the reference (its ukernels are separate calls): mmt4d
 * whose result goes straight into a row-major out_size0 x out_size1 matrix,
 * `out_stride0` elements between rows. Equal, bit for bit, to iree_uk_mmt4d
 * into a tiled [M][N][M0][N0] temporary followed by iree_uk_unpack of it
 * without transposes (tools/unpack_test.c:13-58 is the index map), minus the
 * temporary's HBM round trip. With IREE_UK_FLAG_MMT4D_ACCUMULATE the matrix is
 * also the accumulator input. Operand arguments, tile sizes and flags are
 * those of iree_uk_mmt4d; out_size0 <= M*M0 and out_size1 <= N*N0 (the rest of
 * the last tiles is dropped). */
typedef struct iree_uk_amd_mmt4d_unpack_params_t {
  const void* lhs_buffer;
  iree_uk_index_t lhs_offset;
  iree_uk_index_t lhs_stride0;
  const void* rhs_buffer;
  iree_uk_index_t rhs_offset;
  iree_uk_index_t rhs_stride0;
  void* out_buffer;
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t out_size0;
  iree_uk_index_t out_size1;
  iree_uk_index_t M;
  iree_uk_index_t N;
  iree_uk_index_t K;
  int32_t M0;
  int32_t N0;
  int32_t K0;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_amd_mmt4d_unpack_params_t;

IREE_UK_AMD_EXPORT void iree_uk_amd_mmt4d_unpack(
    const void* lhs_buffer, iree_uk_index_t lhs_offset,
    iree_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0, void* out_buffer,
    iree_uk_index_t out_offset, iree_uk_index_t out_stride0,
    iree_uk_index_t out_size0, iree_uk_index_t out_size1, iree_uk_index_t M,
    iree_uk_index_t N, iree_uk_index_t K, int32_t M0, int32_t N0, int32_t K0,
    uint32_t flags, const uint64_t* cpu_data);
IREE_UK_AMD_EXPORT void iree_uk_amd_mmt4d_unpack_p(
    const iree_uk_amd_mmt4d_unpack_params_t* params);

/*===----------------------------------------------------------------------===*/
/* Fused mmt4d + dequantizing unpack                                           */
/*===----------------------------------------------------------------------===*/

/* No counterpart in the reference (a quantized linear layer there is mmt4d,
 * unpack and a compiler-generated elementwise dispatch): mmt4d of a type with
 * a 32-bit accumulator (s32 or f32 out type), whose result goes into a
 * row-major f32 out_size0 x out_size1 matrix as
 *
 *   out[i][j] = (float)(acc0[i][j] + sum_k lhs[i][k] * rhs[j][k])
 *               * row_scale[i] * col_scale[j]
 *
 * evaluated in f32 from left to right (convert, multiply by the row scale,
 * multiply by the column scale). `row_scale` has out_size0 and `col_scale`
 * out_size1 f32 entries; either may be NULL and then reads as 1. acc0 is 0, or
 * with IREE_UK_FLAG_MMT4D_ACCUMULATE the tiled [M][N][M0][N0] buffer
 * `acc_buffer` of the mmt4d out type (`acc_offset` and `acc_stride0` in
 * elements, as out_offset / out_stride0 of iree_uk_mmt4d), which is only read.
 * For the integer types the result equals, bit for bit, iree_uk_mmt4d into the
 * accumulator buffer, iree_uk_unpack and the scaling above. Unlike
 * iree_uk_mmt4d, K == 0 with ACCUMULATE still writes the (scaled) matrix.
 * Operand arguments, tile sizes and flags are otherwise those of
 * iree_uk_mmt4d; out_size0 <= M*M0 and out_size1 <= N*N0. */
typedef struct iree_uk_amd_mmt4d_dequant_unpack_params_t {
  const void* lhs_buffer;
  iree_uk_index_t lhs_offset;
  iree_uk_index_t lhs_stride0;
  const void* rhs_buffer;
  iree_uk_index_t rhs_offset;
  iree_uk_index_t rhs_stride0;
  const void* acc_buffer;
  iree_uk_index_t acc_offset;
  iree_uk_index_t acc_stride0;
  void* out_buffer;
  iree_uk_index_t out_offset;
  iree_uk_index_t out_stride0;
  iree_uk_index_t out_size0;
  iree_uk_index_t out_size1;
  const float* row_scale;
  const float* col_scale;
  iree_uk_index_t M;
  iree_uk_index_t N;
  iree_uk_index_t K;
  int32_t M0;
  int32_t N0;
  int32_t K0;
  uint32_t flags;
  const uint64_t* cpu_data;
} iree_uk_amd_mmt4d_dequant_unpack_params_t;

IREE_UK_AMD_EXPORT void iree_uk_amd_mmt4d_dequant_unpack(
    const void* lhs_buffer, iree_uk_index_t lhs_offset,
    iree_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_uk_index_t rhs_offset, iree_uk_index_t rhs_stride0,
    const void* acc_buffer, iree_uk_index_t acc_offset,
    iree_uk_index_t acc_stride0, void* out_buffer, iree_uk_index_t out_offset,
    iree_uk_index_t out_stride0, iree_uk_index_t out_size0,
    iree_uk_index_t out_size1, const float* row_scale, const float* col_scale,
    iree_uk_index_t M, iree_uk_index_t N, iree_uk_index_t K, int32_t M0,
    int32_t N0, int32_t K0, uint32_t flags, const uint64_t* cpu_data);
IREE_UK_AMD_EXPORT void iree_uk_amd_mmt4d_dequant_unpack_p(
    const iree_uk_amd_mmt4d_dequant_unpack_params_t* params);

/*===----------------------------------------------------------------------===*/
/* HAL executable plugin face                                                  */
/*===----------------------------------------------------------------------===*/

/* The library is also a HAL executable plugin: an IREE runtime started with
 * `--executable_plugin=<path to this library>`
 * (runtime/src/iree/tooling/context_util.c:589-614) looks this symbol up
 * (runtime/src/iree/hal/local/executable_plugin.h:185-191, export name :188-189)
 * and resolves the imports `iree_uk_mmt4d`, `iree_uk_pack` and `iree_uk_unpack`
 * of compiled LLVMCPU programs through it. The result is the reference's
 * `const iree_hal_executable_plugin_header_t**` (interface version 0.1,
 * executable_plugin.h:404-461), or NULL when `max_version` is below 0.1. Each
 * resolved import is an `int fn(void* params_ptr, void* context, void*
 * reserved)` thunk (runtime/src/iree/hal/local/executable_library.h:150-158)
 * that forwards to the `_p` entry points above and returns non-zero when the
 * call failed. */
IREE_UK_AMD_EXPORT const void* iree_hal_executable_plugin_query(
    uint32_t max_version, void* reserved);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* IREE_UK_AMD_H_ */
