/*
 * rtat_oracle.h — CPU restatement of the reference's execution path.  TEST INFRASTRUCTURE:
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may link or call it;
 * nothing under rtatblas_amd/ does.
 *
 * Two layers, as in the reference:
 *   1. the four BLAS-3 calls it delegates to (src/matrix_ops/matrixop.h:15-140), restated as
 *      plain loops with the semantics of the vendor routines it binds (hipBLAS);
 *   2. the lazy matrix-op tree and the per-routine variants built on top of them
 *      (src/matrix_ops/matrixop.h:142-617, src/methods/{gemm,syrk,trsm}.cpp), including the
 *      workspace accounting of matrixop.h:164-185.
 *
 * Enum values are the hipBLAS ones (op N/T = 111/112, fill upper/lower = 121/122,
 * diag non-unit/unit = 131/132, side left/right = 141/142).  All matrices column-major.
 */
#ifndef RTAT_ORACLE_H
#define RTAT_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_OP_N = 111, ORC_OP_T = 112, ORC_UPPER = 121, ORC_LOWER = 122, ORC_NON_UNIT = 131,
       ORC_UNIT = 132, ORC_LEFT = 141, ORC_RIGHT = 142 };

/* ---- layer 1: the BLAS calls ------------------------------------------------------- */
void orc_dgemm(int transa, int transb, int m, int n, int k, double alpha, const double* A,
               int lda, const double* B, int ldb, double beta, double* C, int ldc);
void orc_dsyrk(int uplo, int trans, int n, int k, double alpha, const double* A, int lda,
               double beta, double* C, int ldc);
void orc_dtrsm(int side, int uplo, int trans, int diag, int m, int n, double alpha,
               const double* A, int lda, double* B, int ldb);
void orc_dgeam(int transa, int transb, int m, int n, double alpha, const double* A, int lda,
               double beta, const double* B, int ldb, double* C, int ldc);

/* Route orc_dgemm / orc_dsyrk / orc_dtrsm through a host CBLAS found by dlopen (path may be
 * NULL to search the usual places).  Returns the number of threads it will use, 0 when no
 * library was found (the plain loops stay in use).  Used for large sizes and as the CPU
 * baseline; orc_cblas_off() restores the loops. */
int orc_cblas_on(const char* path);
void orc_cblas_off(void);
const char* orc_cblas_name(void);

/* ---- operand generator (same function as rtat_dfill on the device) ------------------ */
/* kind: 0 iid [-1,1), 1 symmetric, 2 well-conditioned lower triangular (strict upper NaN),
 * 3 uniform (0,1], 4 the lower triangle of kind 2 mirrored to the upper.  Padding rows m..ld-1 are set to NaN. */
void orc_dfill(double* A, int m, int n, int ld, uint64_t seed, int kind);

/* ---- layer 2: variants = trees over layer 1 ---------------------------------------- */
/* Variant strings are the reference's: GEMM "[ta][tb][tc]" N/T (gemm.cpp:147-157), GEMM_Pad
 * "[ta][tb][tc][pa][pb][pc]" N/T and N/P (gemm.cpp:41-53), SYRK "[tA][tC]" T/F
 * (syrk.cpp:37-46), TRSM "[swap][tA]" T/F (trsm.cpp:38-47).
 * Each *_workspace returns the bytes the variant needs (Executor::calculate_workspace,
 * executor.h:41-44); each *_variant runs it with `ws` as scratch and returns 0, or -1 when
 * the variant string is malformed, -2 when ws_bytes is short (executor.h:49-51). */
long orc_gemm_workspace(const char* variant, int transa, int transb, int m, int n, int k,
                        int lda, int ldb, int ldc);
int orc_gemm_variant(const char* variant, int transa, int transb, int m, int n, int k,
                     double alpha, const double* A, int lda, const double* B, int ldb,
                     double beta, double* C, int ldc, void* ws, size_t ws_bytes);
long orc_syrk_workspace(const char* variant, int uplo, int trans, int n, int k, int lda, int ldc);
int orc_syrk_variant(const char* variant, int uplo, int trans, int n, int k, double alpha,
                     const double* A, int lda, double beta, double* C, int ldc, void* ws,
                     size_t ws_bytes);
long orc_trsm_workspace(const char* variant, int side, int uplo, int trans, int diag, int m,
                        int n, int lda, int ldb);
int orc_trsm_variant(const char* variant, int side, int uplo, int trans, int diag, int m, int n,
                     double alpha, const double* A, int lda, double* B, int ldb, void* ws,
                     size_t ws_bytes);

#ifdef __cplusplus
}
#endif
#endif
