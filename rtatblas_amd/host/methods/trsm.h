// TRSM call descriptor, problem key and variants (reference src/methods/trsm.h).
#pragma once
#include <executor.h>
#include <matrixop.h>

#include <string>
#include <vector>

#include "base_options.h"
#include "spelled.h"

namespace rtat {

// Solve op(A) X = alpha B (left) or X op(A) = alpha B (right), X overwriting B (reference
// trsm.h:10-33).
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

// Spelled "side,uplo,trans,diag,m,n" (reference trsm.cpp:8-18).
struct TRSM_Key : Spelled_Once<TRSM_Key> {
  const BLAS_Side side;
  const BLAS_Fill_Mode uplo;
  const BLAS_Operation trans;
  const BLAS_Diag diag;
  const int m, n;

  TRSM_Key(BLAS_Side side, BLAS_Fill_Mode uplo, BLAS_Operation trans, BLAS_Diag diag, int m, int n)
      : Spelled_Once(spell(side, uplo, trans, diag, m, n)), side(side), uplo(uplo), trans(trans),
        diag(diag), m(m), n(n) {}
  template <typename T>
  TRSM_Key(TRSM_Inputs<T> in)
      : TRSM_Key(in.side, in.uplo, in.trans, in.diag, (int)in.m(), (int)in.n()) {}

  double flopcount() const {
    return side == gpu::BLAS_SIDE_LEFT ? (double)m * m * n : (double)m * n * n;
  }

 private:
  static std::string spell(BLAS_Side, BLAS_Fill_Mode, BLAS_Operation, BLAS_Diag, int m, int n);
};

// Variant "[swap][tA]": solve the transposed system on the other side / transpose A first
// (reference trsm.h:59-82).
struct TRSM_Options : Switch_Variant<TRSM_Options> {
  Bool_Op swap_side, transpose_A;

  TRSM_Options() = default;
  TRSM_Options(Bool_Op swap_side, Bool_Op transpose_A)
      : swap_side(swap_side), transpose_A(transpose_A) {}
  auto switches() { return std::tie(swap_side, transpose_A); }
  auto switches() const { return std::tie(swap_side, transpose_A); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(TRSM_Inputs<T>);
};

// Variant "[swap][tA]" with swap in F / T / X: TRSM_Options plus the fused form of swap_side
// (Fusable_Op, base_options.h).  The panel solve takes its slab of right-hand sides along
// either dimension of B, so the solve of the transposed system on the other side is the solve
// in place: "X?" is one TRSM on B, without B^T in scratch and without the transposing
// write-back of the tree (reference trsm.cpp:86-103).  That is the tree of "F?", so "X?" can
// be asked for by name but is not enumerated beside it.
struct TRSM_Options_Fused : Switch_Variant<TRSM_Options_Fused> {
  Fusable_Bool_Op swap_side;
  Bool_Op transpose_A;

  TRSM_Options_Fused() = default;
  TRSM_Options_Fused(Fusable_Bool_Op swap_side, Bool_Op transpose_A)
      : swap_side(swap_side), transpose_A(transpose_A) {}
  auto switches() { return std::tie(swap_side, transpose_A); }
  auto switches() const { return std::tie(swap_side, transpose_A); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(TRSM_Inputs<T>);
};

// Variant "[swap][tA]/<tile>/<tail>/<panel>": the reference's switches (trsm.cpp:29-36)
// jointly with the kernel's own choices - tile shape and tail mode of the trailing GEMM
// updates and the height of the panel solves (512 or 1024 rows per launch) - which the
// library otherwise settles by rules fitted to one part.  180 settings; "FF/auto/auto/auto" is
// the plain call.
struct TRSM_Options_Tile : Switch_Variant<TRSM_Options_Tile> {
  Bool_Op swap_side, transpose_A;
  Tile_Op tile;
  Tail_Op tail;
  Panel_Op panel;

  TRSM_Options_Tile() = default;
  TRSM_Options_Tile(Bool_Op swap_side, Bool_Op transpose_A, Tile_Op tile, Tail_Op tail,
                    Panel_Op panel)
      : swap_side(swap_side), transpose_A(transpose_A), tile(tile), tail(tail), panel(panel) {}
  auto switches() { return std::tie(swap_side, transpose_A, tile, tail, panel); }
  auto switches() const { return std::tie(swap_side, transpose_A, tile, tail, panel); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(TRSM_Inputs<T>);
};

namespace detail {
template <typename T>
void warm_trsm_kernels(gpu::blasHandle_t handle);
}

template <typename T>
using TRSM_Executor =
    Warmed_Executor<TRSM_Inputs<T>, TRSM_Key, TRSM_Options, &detail::warm_trsm_kernels<T>>;

template <typename T>
using TRSM_Executor_Fused = Warmed_Executor<TRSM_Inputs<T>, TRSM_Key, TRSM_Options_Fused,
                                            &detail::warm_trsm_kernels<T>>;

template <typename T>
using TRSM_Executor_Tile =
    Warmed_Executor<TRSM_Inputs<T>, TRSM_Key, TRSM_Options_Tile, &detail::warm_trsm_kernels<T>>;

}  // namespace rtat
