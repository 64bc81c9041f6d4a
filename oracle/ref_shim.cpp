// extern "C" doors onto the REFERENCE's own executors, compiled from the reference's sources
// (oracle/Makefile) in two builds:
//   ref         -> _ref/librtat_ref.so         the reference as it ships, linked against hipBLAS:
//                                              "the reference built on hipBLAS";
//   ref_native  -> _ref/librtat_ref_native.so  the same sources with the BLAS alias block of its
//                                              gpu-api.h rebound to the rtat_* entry points of
//                                              include/rtat_native.h and linked against
//                                              librtat_native.so instead of hipBLAS: the drop-in.
// TEST INFRASTRUCTURE: loaded only by tests/ and by bench.py's reference timing leg, only
// when the libraries exist.  Only gpu:: names are used here, so the file serves both builds.
//
// Nothing of the reference is restated here: every call goes through its GEMM_Executor /
// SYRK_Executor / TRSM_Executor (src/methods/executor.h:18-33), i.e. form_operation ->
// MatrixOp::execute -> gpuT* -> gpu::blasD*.  Matrices are device pointers.
#include <gemm.h>
#include <syrk.h>
#include <trsm.h>

#include <cstring>
#include <string>

using namespace rtat;

namespace {

struct Ctx {
  gpu::blasHandle_t handle = nullptr;
  GEMM_Executor<double> gemm;
  GEMM_Executor_Pad<double> gemm_pad;
  SYRK_Executor<double> syrk;
  TRSM_Executor<double> trsm;
  Ctx() { gpu::blasCreate(&handle); }
};

Ctx& ctx() {
  static Ctx c;
  return c;
}

Matrix<double> view(const double* p, size_t m, size_t n, size_t ld) {
  return Matrix<double>(Workspace(const_cast<double*>(p), ld * n), m, n, ld);
}

BLAS_Op op_atom(char c) { return BLAS_Op(std::string(1, c)); }
Pad_Op pad_atom(char c) { return Pad_Op(std::string(1, c)); }
Bool_Op bool_atom(char c) { return Bool_Op(std::string(1, c)); }

GEMM_Inputs<double> gemm_in(int ta, int tb, int m, int n, int k, double alpha, const double* A,
                            int lda, const double* B, int ldb, double beta, double* C, int ldc) {
  const bool at = ta == gpu::BLAS_OP_T, bt = tb == gpu::BLAS_OP_T;
  return GEMM_Inputs<double>(ctx().handle, BLAS_Operation((gpu::blasOperation_t)ta),
                             BLAS_Operation((gpu::blasOperation_t)tb),
                             view(A, at ? k : m, at ? m : k, lda),
                             view(B, bt ? n : k, bt ? k : n, ldb), view(C, m, n, ldc), alpha, beta);
}

// Last timing the executor logged for (key, opts): blocks on its events.
template <class Exec, class Key, class Opts>
float last_ms(Exec& e, Key key, Opts opts) {
  auto& bank = e.get_timings(key)[opts];
  bank.synchronize();
  const auto& ts = bank.get_times();
  return ts.empty() ? -1.f : ts.back();
}

}  // namespace

extern "C" {

// 1 when the BLAS boundary of this build is librtat_native, 0 when it is hipBLAS.
int ref_on_native(void) {
#ifdef RTAT_REF_ON_NATIVE
  return 1;
#else
  return 0;
#endif
}

// All functions return 0 on success, -1 on a malformed variant, -2 on any exception.

long long ref_gemm_workspace(const char* v, int ta, int tb, int m, int n, int k, int lda, int ldb,
                             int ldc) {
  try {
    auto in = gemm_in(ta, tb, m, n, k, 1.0, nullptr, lda, nullptr, ldb, 0.0, nullptr, ldc);
    if (std::strlen(v) == 3)
      return (long long)ctx().gemm.calculate_workspace(
          in, GEMM_Options(op_atom(v[0]), op_atom(v[1]), op_atom(v[2])));
    if (std::strlen(v) == 6)
      return (long long)ctx().gemm_pad.calculate_workspace(
          in, GEMM_Options_Pad(op_atom(v[0]), pad_atom(v[3]), op_atom(v[1]), pad_atom(v[4]),
                               op_atom(v[2]), pad_atom(v[5])));
    return -1;
  } catch (...) {
    return -2;
  }
}

int ref_gemm(const char* v, int ta, int tb, int m, int n, int k, double alpha, const double* A,
             int lda, const double* B, int ldb, double beta, double* C, int ldc, void* ws,
             size_t ws_bytes, void* stream, float* ms) {
  try {
    gpu::blasSetStream(ctx().handle, (hipStream_t)stream);
    Stream s((hipStream_t)stream);
    auto in = gemm_in(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
    Workspace space((char*)ws, ws_bytes);
    if (std::strlen(v) == 3) {
      GEMM_Options o(op_atom(v[0]), op_atom(v[1]), op_atom(v[2]));
      ctx().gemm.execute(in, o, space, s);
      if (ms) *ms = last_ms(ctx().gemm, GEMM_Key(in), o);
    } else if (std::strlen(v) == 6) {
      GEMM_Options_Pad o(op_atom(v[0]), pad_atom(v[3]), op_atom(v[1]), pad_atom(v[4]),
                         op_atom(v[2]), pad_atom(v[5]));
      ctx().gemm_pad.execute(in, o, space, s);
      if (ms) *ms = last_ms(ctx().gemm_pad, GEMM_Key(in), o);
    } else {
      return -1;
    }
    return 0;
  } catch (...) {
    return -2;
  }
}

int ref_syrk(const char* v, int uplo, int trans, int n, int k, double alpha, const double* A,
             int lda, double beta, double* C, int ldc, void* ws, size_t ws_bytes, void* stream,
             float* ms) {
  try {
    if (std::strlen(v) != 2) return -1;
    gpu::blasSetStream(ctx().handle, (hipStream_t)stream);
    Stream s((hipStream_t)stream);
    const bool t = trans == gpu::BLAS_OP_T;
    SYRK_Inputs<double> in(ctx().handle, BLAS_Fill_Mode((gpu::blasFillMode_t)uplo),
                           BLAS_Operation((gpu::blasOperation_t)trans),
                           view(A, t ? k : n, t ? n : k, lda), view(C, n, n, ldc), alpha, beta);
    SYRK_Options o(bool_atom(v[0]), bool_atom(v[1]));
    ctx().syrk.execute(in, o, Workspace((char*)ws, ws_bytes), s);
    if (ms) *ms = last_ms(ctx().syrk, SYRK_Key(in), o);
    return 0;
  } catch (...) {
    return -2;
  }
}

int ref_trsm(const char* v, int side, int uplo, int trans, int diag, int m, int n, double alpha,
             const double* A, int lda, double* B, int ldb, void* ws, size_t ws_bytes, void* stream,
             float* ms) {
  try {
    if (std::strlen(v) != 2) return -1;
    gpu::blasSetStream(ctx().handle, (hipStream_t)stream);
    Stream s((hipStream_t)stream);
    const size_t na = side == gpu::BLAS_SIDE_LEFT ? m : n;
    TRSM_Inputs<double> in(ctx().handle, BLAS_Side((gpu::blasSideMode_t)side),
                           BLAS_Fill_Mode((gpu::blasFillMode_t)uplo),
                           BLAS_Operation((gpu::blasOperation_t)trans),
                           BLAS_Diag((gpu::blasDiagType_t)diag), view(A, na, na, lda),
                           view(B, m, n, ldb), alpha);
    TRSM_Options o(bool_atom(v[0]), bool_atom(v[1]));
    ctx().trsm.execute(in, o, Workspace((char*)ws, ws_bytes), s);
    if (ms) *ms = last_ms(ctx().trsm, TRSM_Key(in), o);
    return 0;
  } catch (...) {
    return -2;
  }
}

// The reference's geam call (MatrixMove / MatrixAccumulate go through it): B-sized m x n.
int ref_geam(int ta, int tb, int m, int n, double alpha, const double* A, int lda, double beta,
             const double* B, int ldb, double* C, int ldc, void* stream) {
  gpu::blasSetStream(ctx().handle, (hipStream_t)stream);
  return (int)gpu::blasDgeam(ctx().handle, (gpu::blasOperation_t)ta, (gpu::blasOperation_t)tb, m, n,
                             &alpha, A, lda, &beta, B, ldb, C, ldc);
}

}  // extern "C"
