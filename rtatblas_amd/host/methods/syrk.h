// SYRK call descriptor, problem key and variants (reference src/methods/syrk.h).
#pragma once
#include <executor.h>
#include <matrixop.h>

#include <string>
#include <vector>

#include "base_options.h"
#include "spelled.h"

namespace rtat {

// The `uplo` triangle of C = alpha op(A) op(A)^T + beta C (reference syrk.h:10-30).
template <typename T>
struct SYRK_Inputs {
  using Scalar = T;

  gpu::blasHandle_t handle;
  BLAS_Fill_Mode uplo;
  BLAS_Operation trans;
  const Matrix<T> A;
  Matrix<T> C;
  const T alpha, beta;

  SYRK_Inputs(gpu::blasHandle_t handle, BLAS_Fill_Mode uplo, BLAS_Operation trans,
              const Matrix<T> A, Matrix<T> C, T alpha, T beta)
      : handle(handle), uplo(uplo), trans(trans), A(A), C(C), alpha(alpha), beta(beta) {}

  size_t n() const { return C.dims().m; }
  size_t k() const { return trans == gpu::BLAS_OP_N ? A.dims().n : A.dims().m; }
};

// Spelled "uplo,trans,n,k" (reference syrk.cpp:8-17).
struct SYRK_Key : Spelled_Once<SYRK_Key> {
  const BLAS_Fill_Mode uplo;
  const BLAS_Operation trans;
  const int n, k;

  SYRK_Key(BLAS_Fill_Mode uplo, BLAS_Operation trans, int n, int k)
      : Spelled_Once(spell(uplo, trans, n, k)), uplo(uplo), trans(trans), n(n), k(k) {}
  template <typename T>
  SYRK_Key(SYRK_Inputs<T> in) : SYRK_Key(in.uplo, in.trans, (int)in.n(), (int)in.k()) {}

  double flopcount() const { return (double)n * (n + 1.0) * k; }

 private:
  static std::string spell(BLAS_Fill_Mode uplo, BLAS_Operation trans, int n, int k);
};

// Variant "[tA][tC]": transpose A first / compute the other triangle into scratch and add it
// back transposed (reference syrk.h:54-77).
struct SYRK_Options : Switch_Variant<SYRK_Options> {
  Bool_Op transpose_A, transpose_C;

  SYRK_Options() = default;
  SYRK_Options(Bool_Op transpose_A, Bool_Op transpose_C)
      : transpose_A(transpose_A), transpose_C(transpose_C) {}
  auto switches() { return std::tie(transpose_A, transpose_C); }
  auto switches() const { return std::tie(transpose_A, transpose_C); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(SYRK_Inputs<T>);
};

// Variant "[tA][tC]" with tC in F / T / X: SYRK_Options plus the fused form of transpose_C
// (Fusable_Op, base_options.h).  The product is symmetric, so the opposite triangle added
// back transposed is the wanted triangle computed in place: "?X" is one SYRK launch on C, no
// zeroed n x n scratch and no accumulate pass, and - unlike "?T" (reference syrk.cpp:83-97) -
// it leaves the triangle the caller did not ask for untouched.  That is the tree of "?F", so
// "?X" can be asked for by name but is not enumerated beside it.
struct SYRK_Options_Fused : Switch_Variant<SYRK_Options_Fused> {
  Bool_Op transpose_A;
  Fusable_Bool_Op transpose_C;

  SYRK_Options_Fused() = default;
  SYRK_Options_Fused(Bool_Op transpose_A, Fusable_Bool_Op transpose_C)
      : transpose_A(transpose_A), transpose_C(transpose_C) {}
  auto switches() { return std::tie(transpose_A, transpose_C); }
  auto switches() const { return std::tie(transpose_A, transpose_C); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(SYRK_Inputs<T>);
};

// Variant "[tA][tC]/<tile>/<tail>": the reference's switches (syrk.cpp:28-35) jointly with the
// kernel's own choices - the macro-tile shape of the MFMA core and what happens to the tiles
// of the last partial round (computed whole, or cut along K) - which the library otherwise
// settles by a rule fitted to one part.  60 settings; "FF/auto/auto" is the plain call.
struct SYRK_Options_Tile : Switch_Variant<SYRK_Options_Tile> {
  Bool_Op transpose_A, transpose_C;
  Tile_Op tile;
  Tail_Op tail;

  SYRK_Options_Tile() = default;
  SYRK_Options_Tile(Bool_Op transpose_A, Bool_Op transpose_C, Tile_Op tile, Tail_Op tail)
      : transpose_A(transpose_A), transpose_C(transpose_C), tile(tile), tail(tail) {}
  auto switches() { return std::tie(transpose_A, transpose_C, tile, tail); }
  auto switches() const { return std::tie(transpose_A, transpose_C, tile, tail); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(SYRK_Inputs<T>);
};

namespace detail {
template <typename T>
void warm_syrk_kernels(gpu::blasHandle_t handle);
}

template <typename T>
using SYRK_Executor =
    Warmed_Executor<SYRK_Inputs<T>, SYRK_Key, SYRK_Options, &detail::warm_syrk_kernels<T>>;

template <typename T>
using SYRK_Executor_Fused = Warmed_Executor<SYRK_Inputs<T>, SYRK_Key, SYRK_Options_Fused,
                                            &detail::warm_syrk_kernels<T>>;

template <typename T>
using SYRK_Executor_Tile =
    Warmed_Executor<SYRK_Inputs<T>, SYRK_Key, SYRK_Options_Tile, &detail::warm_syrk_kernels<T>>;

}  // namespace rtat
