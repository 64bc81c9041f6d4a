// SYRK call descriptor, key and variants (reference src/methods/syrk.h).
#pragma once
#include <executor.h>
#include <matrixop.h>

#include <string>
#include <vector>

#include "base_options.h"

namespace rtat {

// uplo triangle of C = alpha op(A) op(A)^T + beta C.
template <typename T>
struct SYRK_Inputs {
  using Scalar = T;

  gpu::blasHandle_t handle;
  BLAS_Fill_Mode uplo;
  BLAS_Operation trans;
  const Matrix<T> A;
  Matrix<T> C;
  const T alpha;
  const T beta;

  SYRK_Inputs(gpu::blasHandle_t handle, BLAS_Fill_Mode uplo, BLAS_Operation trans,
              const Matrix<T> A, Matrix<T> C, T alpha, T beta)
      : handle(handle), uplo(uplo), trans(trans), A(A), C(C), alpha(alpha), beta(beta) {}

  size_t n() const { return C.dims().m; }
  size_t k() const { return trans == gpu::BLAS_OP_N ? A.dims().n : A.dims().m; }
};

// Ordered by its string "uplo,trans,n,k" (reference syrk.cpp:8-17).
struct SYRK_Key {
  BLAS_Fill_Mode uplo;
  BLAS_Operation trans;
  int n;
  int k;

  SYRK_Key(BLAS_Fill_Mode uplo, BLAS_Operation trans, int n, int k)
      : uplo(uplo), trans(trans), n(n), k(k) {}
  template <typename T>
  SYRK_Key(SYRK_Inputs<T> i) : SYRK_Key(i.uplo, i.trans, (int)i.n(), (int)i.k()) {}

  operator std::string() const;
  bool operator<(const SYRK_Key&) const;
  friend std::ostream& operator<<(std::ostream&, const SYRK_Key&);
  double flopcount() const { return (double)n * (n + 1.0) * k; }
};

// Variant "[tA][tC]": transpose A first / compute the other triangle into scratch and add
// it back transposed.
struct SYRK_Options {
  Bool_Op transpose_A;
  Bool_Op transpose_C;

  SYRK_Options() = default;
  SYRK_Options(Bool_Op transpose_A, Bool_Op transpose_C)
      : transpose_A(transpose_A), transpose_C(transpose_C) {}

  static SYRK_Options default_opts() { return SYRK_Options(); }
  static std::vector<SYRK_Options> enumerate();
  operator std::string() const;
  bool operator<(const SYRK_Options&) const;
  friend std::ostream& operator<<(std::ostream&, const SYRK_Options);
  friend std::istream& operator>>(std::istream&, SYRK_Options&);

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(SYRK_Inputs<T>);
};

namespace detail {
template <typename T>
void warm_syrk_kernels(gpu::blasHandle_t handle);
}

template <typename T>
class SYRK_Executor : public Executor<SYRK_Inputs<T>, SYRK_Key, SYRK_Options> {
 protected:
  void warmup(SYRK_Inputs<T> params, SYRK_Options, Stream) override {
    detail::warm_syrk_kernels<T>(params.handle);
  }
};

}  // namespace rtat
