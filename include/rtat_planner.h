/*
 * rtat_planner.h — C ABI of the layer above the BLAS boundary: the variant trees and the
 * autotuning planner, for callers that cannot include the C++ headers (other languages,
 * ctypes).  Each entry point is a thin door onto the C++ classes that mirror the reference:
 *
 *   rtat_planner_create("gemm" | "gemm_pad" | "gemm_tile" | "gemm_pad_tile" | "gemm_fused" |
 *                       "syrk" | "syrk_tile" | "syrk_fused" | "trsm" | "trsm_tile" | "trsm_fused")
 *        Planning_System<GEMM_Executor<double>> ... (reference src/rtat.h:20-60,
 *        src/planning/planning_system.h:38-131; method names as in src/app/test_harness.h:56-66)
 *   rtat_planner_{gemm,syrk,trsm}
 *        create_plan (planning_system.h:65-96) when `variant` is NULL, then
 *        Planning_System::execute (planning_system.h:102-114) with the caller's workspace
 *   rtat_planner_*_workspace
 *        Planning_System::calculate_workspace (planning_system.h:116-118)
 *   rtat_planner_stats_json
 *        make_statistics().json() (planner_statistics.h:50-67)
 *
 * All calls are fp64, enqueue on the stream of `handle`, and never throw: errors come back
 * as negative return values with a message readable through rtat_planner_last_error().
 * Variant strings are the reference's: "NNN".."TTT" (gemm), six letters (gemm_pad), "FF".."TT"
 * (syrk, trsm).  The *_tile methods append the kernel's own choices, each behind a slash, as
 * further switches of the same variant (what src/methods/gemm.cpp:28-39, syrk.cpp:28-35 and
 * trsm.cpp:29-36 enumerate, widened by the axes a vendor BLAS hides): the macro-tile shape
 * (rtat_gemm_variant_name), the tail mode (rtat_tail_mode_name) and, for trsm, the panel
 * height (rtat_trsm_panel_name): "NNN/128x64" (gemm_tile), "NNNNPN/128x64/whole"
 * (gemm_pad_tile), "FF/auto/split" (syrk_tile), "FF/256x128/auto/1024" (trsm_tile).  The
 * *_fused methods also accept the letter X for the switch that transposes the result ("NNX",
 * "FX", "XF"): that transposition done by the kernel itself, in one launch and without
 * scratch - which is the plain call, so X is not enumerated beside N / F.
 */
#ifndef RTAT_PLANNER_H
#define RTAT_PLANNER_H
#include "rtat_native.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rtat_planner* rtat_planner_t;

/* NULL on an unknown method name. */
rtat_planner_t rtat_planner_create(const char* method);
void rtat_planner_destroy(rtat_planner_t p);

/* Samples per variant before a plan is committed (default 3) and the statistic variants are
 * ranked by: 0 mean, 1 median (default), 2 minimum. */
int rtat_planner_configure(rtat_planner_t p, int tests_until_converge, int statistic);

/* Run-off before a plan is committed: the variants within `margin` (a fraction, default
 * 0.05) of the fastest each get `extra_tests` more samples (default 6; 0 = commit at once),
 * and so does the default variant when its fastest sample is that close.  A variant with at
 * least as many run-off samples as exploration samples is ranked by the run-off's alone. */
int rtat_planner_set_refinement(rtat_planner_t p, int extra_tests, double margin);
/* Commit rule: variants whose figure is within `margin` (a fraction, default 0.0025) of the
 * fastest, or within the scatter of their own samples up to twice that, count as tied with
 * it; a tie goes to the default variant if it is among them, else to the variant that needs
 * the least workspace.  0 = the bare argmin of the reference
 * (src/planning/planning_system.h:83-93). */
int rtat_planner_set_tie_margin(rtat_planner_t p, double margin);
/* Which variants may be tried (the reference's Option_Filter, planning_system.h:14-35):
 * a comma-separated list of glob patterns over variant names ('?' any character, '*' any run);
 * the default variant is always admitted.  NULL or "" admits everything again. */
int rtat_planner_set_filter(rtat_planner_t p, const char* patterns);
/* The same filter learned from a timing report of this method (the text
 * rtat_planner_stats_json returned, now or in an earlier process): for problems of a class
 * (flags and size bucket) seen in the report, only variants that came within `slack` (a
 * fraction) of the fastest on some problem of that class are admitted.  Returns the number of
 * problems read, or < 0. */
int rtat_planner_learn_filter(rtat_planner_t p, const char* stats_json, double slack);
/* The names of the variants admitted for a problem, one per line, in the order they are
 * explored.  The pointer stays valid until the next call that returns text on this planner. */
const char* rtat_planner_gemm_admitted(rtat_planner_t p, int transa, int transb, int m, int n,
                                       int k);
const char* rtat_planner_syrk_admitted(rtat_planner_t p, int uplo, int trans, int n, int k);
const char* rtat_planner_trsm_admitted(rtat_planner_t p, int side, int uplo, int trans, int diag,
                                       int m, int n);
/* The reference's exploration: one sample per variant, ranked by the mean, no run-off
 * (src/planning/planning_system.h:53-96). */
int rtat_planner_use_reference_defaults(rtat_planner_t p);

/* Number of variants the planner's method enumerates, and the i-th variant's string (copied
 * into out, NUL-terminated, truncated to out_len). */
int rtat_planner_variant_count(rtat_planner_t p);
int rtat_planner_variant_name(rtat_planner_t p, int i, char* out, size_t out_len);

/* Bytes of workspace `variant` needs for the call; negative on error. */
long long rtat_planner_gemm_workspace(rtat_planner_t p, const char* variant, int transa,
                                      int transb, int m, int n, int k, int lda, int ldb, int ldc);
long long rtat_planner_syrk_workspace(rtat_planner_t p, const char* variant, int uplo, int trans,
                                      int n, int k, int lda, int ldc);
long long rtat_planner_trsm_workspace(rtat_planner_t p, const char* variant, int side, int uplo,
                                      int trans, int diag, int m, int n, int lda, int ldb);
/* Largest workspace any variant of the method needs for the call. */
long long rtat_planner_gemm_workspace_max(rtat_planner_t p, int transa, int transb, int m, int n,
                                          int k, int lda, int ldb, int ldc);
long long rtat_planner_syrk_workspace_max(rtat_planner_t p, int uplo, int trans, int n, int k,
                                          int lda, int ldc);
long long rtat_planner_trsm_workspace_max(rtat_planner_t p, int side, int uplo, int trans, int diag,
                                          int m, int n, int lda, int ldb);

/* One call through the planner.  variant == NULL: run the planner's current plan for the
 * problem (exploring until it has converged); otherwise run that fixed variant.  A variant
 * that does not fit `workspace` degrades to the default variant, as in the reference.  The
 * variant actually run is copied into chosen (may be NULL).  Returns 0, or a negative code. */
int rtat_planner_gemm(rtat_planner_t p, rtat_handle_t handle, const char* variant, int transa,
                      int transb, int m, int n, int k, double alpha, const double* A, int lda,
                      const double* B, int ldb, double beta, double* C, int ldc, void* workspace,
                      size_t workspace_bytes, char* chosen, size_t chosen_len);
int rtat_planner_syrk(rtat_planner_t p, rtat_handle_t handle, const char* variant, int uplo,
                      int trans, int n, int k, double alpha, const double* A, int lda, double beta,
                      double* C, int ldc, void* workspace, size_t workspace_bytes, char* chosen,
                      size_t chosen_len);
int rtat_planner_trsm(rtat_planner_t p, rtat_handle_t handle, const char* variant, int side,
                      int uplo, int trans, int diag, int m, int n, double alpha, const double* A,
                      int lda, double* B, int ldb, void* workspace, size_t workspace_bytes,
                      char* chosen, size_t chosen_len);

/* The timing report / the committed plans as JSON text.  The pointer stays valid until the
 * next call of either function on the same planner.  Both synchronise with pending timers. */
const char* rtat_planner_stats_json(rtat_planner_t p);
const char* rtat_planner_plans_json(rtat_planner_t p);
/* Commit plans from the text either function returned earlier; returns how many, or < 0. */
int rtat_planner_load_plans(rtat_planner_t p, const char* json_text);

const char* rtat_planner_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
