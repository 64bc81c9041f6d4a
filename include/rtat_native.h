/*
 * rtat_native.h — C ABI of the MI355X (gfx950) BLAS-3 back end of rtat.
 *
 * This is the boundary the reference crosses in src/gpu-api/gpu-api.h:87-113, where
 * gpu::blasCreate / blasSetStream / blasDgemm / blasDsyrk / blasDtrsm / blasDgeam are
 * aliases of the hipBLAS (or cuBLAS) entry points.  Every function below replaces one of
 * those aliases with a hand-written HIP kernel family; argument order, meaning, integer
 * widths, column-major storage and the host-pointer alpha/beta convention are those of
 * the hipBLAS routines the reference calls, so the four shims in
 * src/matrix_ops/matrixop.h:15-140 bind to them unchanged.
 *
 * Conventions shared by all compute entry points
 *   - matrices are device pointers, column-major, leading dimension in elements;
 *   - alpha/beta are HOST pointers and are read before the call returns;
 *   - work is enqueued on the handle's stream only; nothing synchronises, nothing is
 *     printed, nothing throws: the return value is the only error channel.  One compute
 *     call may allocate: an rtat_dtrsm / rtat_strsm that needs more handle-owned scratch
 *     than any call before it on that handle (one hipMalloc, no synchronisation, no
 *     hipFree; see rtat_set_workspace for how to avoid it);
 *   - with beta == 0 the output is never read (it may hold NaN/Inf);
 *   - m, n or k equal to 0 is legal (quick return / pure scaling);
 *   - enum values are those of hipBLAS so plan files and oracle calls interoperate.
 */
#ifndef RTAT_NATIVE_H
#define RTAT_NATIVE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Opaque per-thread context: stream, device properties, TRSM scratch.
 * Replaces hipblasHandle_t in GEMM_Inputs::handle (src/methods/gemm.h:14). */
typedef struct rtat_native_handle* rtat_handle_t;

/* A hipStream_t passed as an untyped pointer so this header needs no HIP include. */
typedef void* rtat_stream_t;

/* Numeric values equal hipblasStatus_t (hipblas-common.h:39-50); 0 == success, which is
 * all the reference ever tests (src/methods/syrk.h:100). */
typedef enum {
  RTAT_STATUS_SUCCESS = 0,
  RTAT_STATUS_NOT_INITIALIZED = 1,
  RTAT_STATUS_ALLOC_FAILED = 2,
  RTAT_STATUS_INVALID_VALUE = 3,
  RTAT_STATUS_EXECUTION_FAILED = 5,
  RTAT_STATUS_NOT_SUPPORTED = 7,
  RTAT_STATUS_HANDLE_IS_NULLPTR = 9,
  RTAT_STATUS_INVALID_ENUM = 10
} rtat_status_t;

/* gpu::BLAS_OP_N / BLAS_OP_T (src/gpu-api/gpu-api.h:112-113). */
typedef enum { RTAT_OP_N = 111, RTAT_OP_T = 112 } rtat_operation_t;
/* gpu::BLAS_FILL_MODE_UPPER / LOWER (gpu-api.h:110-111). */
typedef enum { RTAT_FILL_UPPER = 121, RTAT_FILL_LOWER = 122 } rtat_fill_t;
/* gpu::BLAS_DIAG_NON_UNIT / UNIT (gpu-api.h:108-109). */
typedef enum { RTAT_DIAG_NON_UNIT = 131, RTAT_DIAG_UNIT = 132 } rtat_diag_t;
/* gpu::BLAS_SIDE_LEFT / RIGHT (gpu-api.h:106-107). */
typedef enum { RTAT_SIDE_LEFT = 141, RTAT_SIDE_RIGHT = 142 } rtat_side_t;

/* ---- handle management ------------------------------------------------------------ */

/* gpu::blasCreate (gpu-api.h:91; callers test_harness.h:149, tests/common.h:17).  Binds the
 * handle to the current device and allocates its 64 MiB of GEMM tail scratch. */
rtat_status_t rtat_create(rtat_handle_t* handle);
/* gpu::blasDestroy (gpu-api.h:92).  Waits for the handle's device (a device-wide
 * synchronisation), then frees handle-owned scratch.  While the handle's stream records into a
 * graph it returns RTAT_STATUS_NOT_SUPPORTED and frees nothing. */
rtat_status_t rtat_destroy(rtat_handle_t handle);
/* gpu::blasSetStream (gpu-api.h:102; test_harness.h:150). All later work goes here. */
rtat_status_t rtat_set_stream(rtat_handle_t handle, rtat_stream_t stream);
/* gpu::blasGetStream (gpu-api.h:101). */
rtat_status_t rtat_get_stream(rtat_handle_t handle, rtat_stream_t* stream);

/* Lend the handle a caller-owned device buffer for TRSM's scratch: the inverted diagonal
 * blocks and the packed off-diagonal blocks of each 512- or 1024-row panel
 * (the role rocBLAS's handle memory plays under hipblasDtrsm).  Pass (NULL, 0) to go back
 * to the handle-owned buffer.  That one grows by hipMalloc when a call needs more than
 * the handle has; a block that is outgrown is kept until rtat_destroy (enqueued work and
 * captured graphs may still name it) and each new block is at least twice the last, so
 * the kept ones never add up to more than the current one.
 * A handle also owns 64 MiB of scratch for the K slices of GEMM / SYRK tail tiles,
 * allocated by rtat_create (if that fails, tails are computed unsplit); while a buffer is
 * lent the library uses no memory of its own and computes tail tiles unsplit (same
 * results up to rounding, a few percent slower on shapes that leave a partial last round
 * of tiles).
 * A handle's scratch serves one stream at a time: let its work drain before rtat_set_stream.
 * While the handle's stream records into a graph nothing is allocated: a TRSM whose
 * scratch is not there yet returns RTAT_STATUS_ALLOC_FAILED and leaves the capture valid
 * (lend a buffer, or run the call once before capturing: the block a captured call used
 * stays valid for every replay until rtat_destroy). */
rtat_status_t rtat_set_workspace(rtat_handle_t handle, void* device_ptr, size_t bytes);
/* Bytes of scratch rtat_dtrsm needs for a given side and size. */
size_t rtat_dtrsm_workspace_bytes(rtat_side_t side, int m, int n);

/* ---- BLAS-3 compute entry points ---------------------------------------------------- */

/* C(m x n) = alpha * op(A) * op(B) + beta * C.
 * Replaces gpu::blasDgemm = hipblasDgemm (gpu-api.h:94), called from
 * gpuTgemm, src/matrix_ops/matrixop.h:24-32. */
rtat_status_t rtat_dgemm(rtat_handle_t handle, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, int k, const double* alpha, const double* A, int lda,
                         const double* B, int ldb, const double* beta, double* C, int ldc);

/* uplo triangle of C(n x n) = alpha * op(A) * op(A)^T + beta * C; the other triangle is
 * not touched.  Replaces gpu::blasDsyrk (gpu-api.h:96), called from gpuTsyrk,
 * matrixop.h:56-63. */
rtat_status_t rtat_dsyrk(rtat_handle_t handle, rtat_fill_t uplo, rtat_operation_t trans, int n,
                         int k, const double* alpha, const double* A, int lda,
                         const double* beta, double* C, int ldc);

/* Solve op(A) X = alpha B (left) or X op(A) = alpha B (right) in place in B(m x n); the
 * triangle of A opposite to uplo (and, for unit diag, the diagonal) is never read.
 * Replaces gpu::blasDtrsm (gpu-api.h:95), called from gpuTtrsm, matrixop.h:87-95. */
rtat_status_t rtat_dtrsm(rtat_handle_t handle, rtat_side_t side, rtat_fill_t uplo,
                         rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                         const double* alpha, const double* A, int lda, double* B, int ldb);

/* rtat_dtrsm for callers that cannot allocate device memory (code under HIP graph capture
 * on a fresh handle, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and result as rtat_dtrsm on a handle with a
 * lent workspace (bit for bit), but the scratch (inverted diagonal blocks, packed panel
 * blocks) is a fixed array inside the library's device image, 18 MiB per GPU, held until
 * the process ends: the call never allocates or frees, whatever the handle has or lacks.
 * Limit: the triangular matrix (m for side left, n for side right) may have order at most
 * RTAT_DTRSM_STATIC_MAX_ORDER, beyond which the call returns RTAT_STATUS_NOT_SUPPORTED and
 * does nothing.  All calls on one GPU, from any handle, share that GPU's array: two such
 * calls whose work overlaps in time on one GPU (different streams) race; calls on one
 * stream are ordered and safe.  GEMM tails inside the solve are computed unsplit. */
#define RTAT_DTRSM_STATIC_MAX_ORDER 4096
rtat_status_t rtat_dtrsm_static(rtat_handle_t handle, rtat_side_t side, rtat_fill_t uplo,
                                rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                                const double* alpha, const double* A, int lda, double* B,
                                int ldb);

/* C(m x n) = alpha * op(A) + beta * op(B): copy, transpose, re-stride (pad), scale,
 * accumulate, zero-fill.  C may alias A (transa == N, lda == ldc) or B (transb == N,
 * ldb == ldc).  An operand whose scalar is 0 is never read.  With alpha == 1, beta == 0
 * the result is a bit-exact copy / transpose.  Replaces gpu::blasDgeam (gpu-api.h:93),
 * called from gpuTgeam, matrixop.h:118-126. */
rtat_status_t rtat_dgeam(rtat_handle_t handle, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, const double* alpha, const double* A, int lda,
                         const double* beta, const double* B, int ldb, double* C, int ldc);

/* Two independent moves C_i(m_i x n_i) = op_i(A_i) - copy, pad copy (re-stride) or transpose,
 * bit-exact - in ONE launch.  What a GEMM variant does to both operands before the multiply:
 * the reference builds it as two MatrixMove nodes, i.e. two geam calls
 * (src/methods/gemm.cpp:98-106, src/matrix_ops/matrixop.h:307-344); this fuses the pair and has
 * no counterpart there.  A_i is m_i x n_i (trans N) or n_i x m_i (trans T) with leading dimension
 * lda; C_i must not overlap A_i or the other job's C.  Either job may be empty (m or n = 0). */
typedef struct rtat_move {
  rtat_operation_t trans;
  int m, n;
  const void* A; /* device pointer, double or float by entry point */
  int lda;
  void* C;
  int ldc;
} rtat_move_t;
rtat_status_t rtat_dmove_pair(rtat_handle_t handle, const rtat_move_t* first,
                              const rtat_move_t* second);
rtat_status_t rtat_smove_pair(rtat_handle_t handle, const rtat_move_t* first,
                              const rtat_move_t* second);

/* Single-precision twins (gpu::blasSgemm/Ssyrk/Strsm/Sgeam, gpu-api.h:97-100) so the
 * float instantiations of the matrix-op tree run at speed: the same kernel templates as the
 * double entry points, on v_mfma_f32_16x16x4_f32 (same tile shapes, AUTO variant). */
rtat_status_t rtat_sgemm(rtat_handle_t handle, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, int k, const float* alpha, const float* A, int lda,
                         const float* B, int ldb, const float* beta, float* C, int ldc);
rtat_status_t rtat_ssyrk(rtat_handle_t handle, rtat_fill_t uplo, rtat_operation_t trans, int n,
                         int k, const float* alpha, const float* A, int lda, const float* beta,
                         float* C, int ldc);
rtat_status_t rtat_strsm(rtat_handle_t handle, rtat_side_t side, rtat_fill_t uplo,
                         rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                         const float* alpha, const float* A, int lda, float* B, int ldb);
rtat_status_t rtat_sgeam(rtat_handle_t handle, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, const float* alpha, const float* A, int lda,
                         const float* beta, const float* B, int ldb, float* C, int ldc);

/* ---- kernel-variant entry points (what src/methods enumerates for the planner) ------ */

/* Kernel variants of the DGEMM core: macro-tile shapes.  RTAT_GEMM_AUTO lets the library
 * pick from the problem shape; the plain entry points above use it.  (For small problems it
 * may pick a 32x32 tile, which has no number of its own: as a fixed choice it would only be
 * a slow one anywhere else.) */
typedef enum {
  RTAT_GEMM_AUTO = 0,
  RTAT_GEMM_T256x128 = 1, /* 256x128x16 macro tile, 8 waves of 64x64, one workgroup per CU */
  RTAT_GEMM_T128x128 = 2, /* 128x128x16 macro tile, 4 waves of 64x64, two per CU          */
  RTAT_GEMM_T128x64 = 3,  /* 128x64x16 macro tile, 4 waves of 64x32 (more, smaller tiles) */
  RTAT_GEMM_T64x64 = 4,   /* 64x64x16 macro tile, 4 waves of 32x32, for small problems    */
  RTAT_GEMM_VARIANT_COUNT = 5
} rtat_gemm_variant_t;

/* Short stable name of a variant ("auto", "256x128", ...); NULL when out of range. */
const char* rtat_gemm_variant_name(int variant);

/* What a launch does with the tiles left over after the last full round of workgroup slots
 * (CUs x workgroups per CU), which would otherwise keep part of the machine busy for a whole
 * tile time. */
typedef enum {
  RTAT_TAIL_AUTO = 0,  /* the library decides (priced by its launch model under RTAT_GEMM_AUTO,
                          a fixed rule for an explicit tile shape)                             */
  RTAT_TAIL_WHOLE = 1, /* every tile computed whole by one workgroup: one launch, no scratch   */
  RTAT_TAIL_SPLIT = 2, /* leftover tiles cut along K wherever two or more slices of at least
                          eight K panels fit; a second small launch sums the slices           */
  RTAT_TAIL_MODE_COUNT = 3
} rtat_tail_mode_t;
/* "auto" / "whole" / "split"; NULL when out of range. */
const char* rtat_tail_mode_name(int mode);

/* Rows of the triangular matrix one launch of the DTRSM panel kernel solves. */
typedef enum {
  RTAT_PANEL_AUTO = 0, /* from the number of right-hand sides and the CU count */
  RTAT_PANEL_512 = 1,  /* four 128-blocks: two workgroups per CU               */
  RTAT_PANEL_1024 = 2, /* eight 128-blocks: one level of GEMM updates fewer    */
  RTAT_PANEL_COUNT = 3
} rtat_trsm_panel_t;
/* "auto" / "512" / "1024"; NULL when out of range. */
const char* rtat_trsm_panel_name(int panel);

/* The `variant` argument of the *_ex entry points is a word of kernel options: the tile
 * shape in bits 0-7 (so a bare rtat_gemm_variant_t is a valid word), the tail mode in bits
 * 8-11, the DTRSM panel height in bits 12-15 (ignored by gemm and syrk).  Any other bit set,
 * or a field out of range, is RTAT_STATUS_INVALID_VALUE. */
#define RTAT_KERNEL_OPTIONS(tile, tail, panel) \
  ((int)(tile) | ((int)(tail) << 8) | ((int)(panel) << 12))
#define RTAT_KERNEL_OPTIONS_TILE(word) ((int)(word) & 0xff)
#define RTAT_KERNEL_OPTIONS_TAIL(word) (((int)(word) >> 8) & 0xf)
#define RTAT_KERNEL_OPTIONS_PANEL(word) (((int)(word) >> 12) & 0xf)

/* rtat_dgemm with explicit kernel options (no counterpart in the reference: it widens the
 * variant space the reference's GEMM_Options enumerate, src/methods/gemm.cpp:28-39,137-145). */
rtat_status_t rtat_dgemm_ex(rtat_handle_t handle, rtat_operation_t transa,
                            rtat_operation_t transb, int m, int n, int k, const double* alpha,
                            const double* A, int lda, const double* B, int ldb,
                            const double* beta, double* C, int ldc, int variant);
/* rtat_dsyrk with explicit kernel options (tile shape, tail mode): the candidates SYRK's
 * variant families enumerate beside the reference's [tA][tC] switches
 * (src/methods/syrk.cpp:28-35). */
rtat_status_t rtat_dsyrk_ex(rtat_handle_t handle, rtat_fill_t uplo, rtat_operation_t trans,
                            int n, int k, const double* alpha, const double* A, int lda,
                            const double* beta, double* C, int ldc, int variant);
/* rtat_dtrsm with explicit kernel options: tile shape and tail mode of its trailing GEMM
 * updates and the panel height of its panel solves - the candidates TRSM's variant families
 * enumerate beside the reference's [swap][tA] switches (src/methods/trsm.cpp:29-36). */
rtat_status_t rtat_dtrsm_ex(rtat_handle_t handle, rtat_side_t side, rtat_fill_t uplo,
                            rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                            const double* alpha, const double* A, int lda, double* B, int ldb,
                            int variant);
/* The single-precision twins of the three calls above. */
rtat_status_t rtat_sgemm_ex(rtat_handle_t handle, rtat_operation_t transa,
                            rtat_operation_t transb, int m, int n, int k, const float* alpha,
                            const float* A, int lda, const float* B, int ldb, const float* beta,
                            float* C, int ldc, int variant);
rtat_status_t rtat_ssyrk_ex(rtat_handle_t handle, rtat_fill_t uplo, rtat_operation_t trans,
                            int n, int k, const float* alpha, const float* A, int lda,
                            const float* beta, float* C, int ldc, int variant);
rtat_status_t rtat_strsm_ex(rtat_handle_t handle, rtat_side_t side, rtat_fill_t uplo,
                            rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                            const float* alpha, const float* A, int lda, float* B, int ldb,
                            int variant);

/* ---- operand generation -------------------------------------------------------------- */

/* Kinds of synthetic operand. */
typedef enum {
  RTAT_FILL_IID = 0,         /* every logical element uniform in [-1, 1)                */
  RTAT_FILL_SYMMETRIC = 1,   /* square: lower triangle as IID, mirrored to the upper    */
  RTAT_FILL_TRI_LOWER = 2,   /* square: (i>j) u/m, diagonal 1+|u|, strict upper = NaN   */
  RTAT_FILL_UNIT_INTERVAL = 3, /* uniform in (0, 1], the range hiprandGenerateUniformDouble has */
  RTAT_FILL_TRI_FULL = 4 /* square: TRI_LOWER's lower triangle mirrored to the upper; either
                            triangle (and the transpose) is a well-conditioned triangular A */
} rtat_fill_kind_t;

/* Deterministic counter-based fill of the logical m x n part of A (ld >= m); element
 * (i, j) depends only on (seed, i, j), never on ld, and the same function exists on the
 * host (oracle).  Rows m..ld-1 of each column are set to NaN so a kernel that reads
 * padding is caught.  Replaces Device_RNG::uniform = hiprandGenerateUniformDouble
 * (gpu-api.h:229-232, used at src/app/test_harness.h:176). */
rtat_status_t rtat_dfill(rtat_handle_t handle, double* A, int m, int n, int ld, uint64_t seed,
                         int kind);
rtat_status_t rtat_sfill(rtat_handle_t handle, float* A, int m, int n, int ld, uint64_t seed,
                         int kind);

/* ---- introspection --------------------------------------------------------------------- */

/* Peaks derived at run time from the device: fp64 matrix flop/s = CUs x clock x 128 and
 * HBM bytes/s = 2 x memory clock x bus width / 8; also the CU count. Any pointer may be NULL. */
rtat_status_t rtat_device_peaks(rtat_handle_t handle, double* fp64_mfma_flops,
                                double* hbm_bytes_per_s, int* compute_units);

/* What the last gemm / syrk call on this handle (or the last trailing update of the last
 * trsm) launched: the tile shape actually used ("32x32" when the automatic choice took the
 * shape that has no variant id), how many leftover tiles were cut along K and into how many
 * slices, and how many were recomputed as 64 x 64 pieces.  For reports that must name the
 * kernel a figure belongs to.  No counterpart in the reference. */
typedef struct rtat_launch_info {
  char tile[16];       /* "256x128" | "128x128" | "128x64" | "64x64" | "32x32" | "" (no launch) */
  int tiles;           /* tiles of that shape the problem has                                */
  int split_tiles;     /* of those, cut along K ...                                          */
  int split_slices;    /* ... into this many slices each (some into one more)                */
  int subdivided;      /* leftover tiles recomputed as 64 x 64 pieces by a second launch     */
  int trsm_panel_rows; /* panel height of the last trsm on the handle (0: none yet)          */
  int trsm_panel_width; /* right-hand sides per workgroup of its panel solves: 16 or 32     */
} rtat_launch_info_t;
rtat_status_t rtat_last_launch(rtat_handle_t handle, rtat_launch_info_t* info);

/* "rtat-native <version> gfx950". */
const char* rtat_version(void);

#ifdef __cplusplus
}
#endif
#endif /* RTAT_NATIVE_H */
