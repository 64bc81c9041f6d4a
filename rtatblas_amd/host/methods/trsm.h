// TRSM call descriptor, key and variants (reference src/methods/trsm.h).
#pragma once
#include <executor.h>
#include <matrixop.h>

#include <string>
#include <vector>

#include "base_options.h"

namespace rtat {

// Solve op(A) X = alpha B (left) or X op(A) = alpha B (right), X overwriting B.
template <typename T>
struct TRSM_Inputs {
  using Scalar = T;

  gpu::blasHandle_t handle;
  BLAS_Side side;
  BLAS_Fill_Mode uplo;
  BLAS_Operation trans;
  BLAS_Diag diag;
  const Matrix<T> A;
  Matrix<T> B;
  const T alpha;

  TRSM_Inputs(gpu::blasHandle_t handle, BLAS_Side side, BLAS_Fill_Mode uplo, BLAS_Operation trans,
              BLAS_Diag diag, const Matrix<T> A, Matrix<T> B, T alpha)
      : handle(handle), side(side), uplo(uplo), trans(trans), diag(diag), A(A), B(B),
        alpha(alpha) {}

  size_t m() const { return B.dims().m; }
  size_t n() const { return B.dims().n; }
};

// Ordered by its string "side,uplo,trans,diag,m,n" (reference trsm.cpp:8-18).
struct TRSM_Key {
  BLAS_Side side;
  BLAS_Fill_Mode uplo;
  BLAS_Operation trans;
  BLAS_Diag diag;
  int m;
  int n;

  TRSM_Key(BLAS_Side side, BLAS_Fill_Mode uplo, BLAS_Operation trans, BLAS_Diag diag, int m, int n)
      : side(side), uplo(uplo), trans(trans), diag(diag), m(m), n(n) {}
  template <typename T>
  TRSM_Key(TRSM_Inputs<T> i) : TRSM_Key(i.side, i.uplo, i.trans, i.diag, (int)i.m(), (int)i.n()) {}

  operator std::string() const;
  bool operator<(const TRSM_Key&) const;
  friend std::ostream& operator<<(std::ostream&, const TRSM_Key&);
  double flopcount() const {
    return side == gpu::BLAS_SIDE_LEFT ? (double)m * m * n : (double)m * n * n;
  }
};

// Variant "[swap][tA]": solve the transposed system on the other side / transpose A first.
struct TRSM_Options {
  Bool_Op swap_side;
  Bool_Op transpose_A;

  TRSM_Options() = default;
  TRSM_Options(Bool_Op swap_side, Bool_Op transpose_A)
      : swap_side(swap_side), transpose_A(transpose_A) {}

  static TRSM_Options default_opts() { return TRSM_Options(); }
  static std::vector<TRSM_Options> enumerate();
  operator std::string() const;
  bool operator<(const TRSM_Options&) const;
  friend std::ostream& operator<<(std::ostream&, const TRSM_Options);
  friend std::istream& operator>>(std::istream&, TRSM_Options&);

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(TRSM_Inputs<T>);
};

namespace detail {
template <typename T>
void warm_trsm_kernels(gpu::blasHandle_t handle);
}

template <typename T>
class TRSM_Executor : public Executor<TRSM_Inputs<T>, TRSM_Key, TRSM_Options> {
 protected:
  void warmup(TRSM_Inputs<T> params, TRSM_Options, Stream) override {
    detail::warm_trsm_kernels<T>(params.handle);
  }
};

}  // namespace rtat
