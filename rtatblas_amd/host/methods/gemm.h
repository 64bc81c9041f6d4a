// GEMM call descriptor, problem key and variant families (reference src/methods/gemm.h).
#pragma once
#include <executor.h>
#include <matrixop.h>

#include <string>
#include <vector>

#include "base_options.h"
#include "spelled.h"

namespace rtat {

// One C = alpha op(A) op(B) + beta C call: handle, op flags, operand views, scalars
// (reference gemm.h:10-31).
template <typename T>
struct GEMM_Inputs {
  using Scalar = T;

  gpu::blasHandle_t handle;
  BLAS_Operation transa, transb;
  const Matrix<T> A, B;
  Matrix<T> C;
  const T alpha, beta;

  GEMM_Inputs(gpu::blasHandle_t handle, BLAS_Operation transa, BLAS_Operation transb,
              const Matrix<T> A, const Matrix<T> B, Matrix<T> C, T alpha, T beta)
      : handle(handle), transa(transa), transb(transb), A(A), B(B), C(C), alpha(alpha),
        beta(beta) {}

  size_t m() const { return C.dims().m; }
  size_t n() const { return C.dims().n; }
  size_t k() const { return transa == gpu::BLAS_OP_N ? A.dims().n : A.dims().m; }
};

// Problem identity for the planner, spelled "ta,tb,,m,k,n" — the doubled comma and the
// (m, k, n) order are the reference's (gemm.cpp:6-16, gemm.h:40), kept so keys sort and print
// the same way.
struct GEMM_Key : Spelled_Once<GEMM_Key> {
  const BLAS_Operation transa, transb;
  const int m, n, k;

  GEMM_Key(BLAS_Operation transa, BLAS_Operation transb, int m, int k, int n)
      : Spelled_Once(spell(transa, transb, m, k, n)), transa(transa), transb(transb), m(m), n(n),
        k(k) {}
  template <typename T>
  GEMM_Key(GEMM_Inputs<T> in)
      : GEMM_Key(in.transa, in.transb, (int)in.m(), (int)in.k(), (int)in.n()) {}

  double flopcount() const { return 2.0 * m * n * k; }

 private:
  static std::string spell(BLAS_Operation ta, BLAS_Operation tb, int m, int k, int n);
};

// Variant "[ta][tb][tc]": which operands get an explicit transpose before / after the
// multiply.  "NNN" is the plain call on the direct-op kernel.  (reference gemm.h:50-80)
struct GEMM_Options : Switch_Variant<GEMM_Options> {
  BLAS_Op transa, transb, transc;

  GEMM_Options() = default;
  GEMM_Options(BLAS_Op transa, BLAS_Op transb, BLAS_Op transc)
      : transa(transa), transb(transb), transc(transc) {}
  auto switches() { return std::tie(transa, transb, transc); }
  auto switches() const { return std::tie(transa, transb, transc); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(GEMM_Inputs<T>);
};

// Variant "[ta][tb][tc][pa][pb][pc]": the transposes plus, per operand, a copy to a leading
// dimension padded to 32 elements — pad-then-multiply versus the masked-edge kernel.  The
// constructor interleaves (ta, pa, tb, pb, tc, pc) as the reference's does (gemm.h:82-111).
struct GEMM_Options_Pad : Switch_Variant<GEMM_Options_Pad> {
  BLAS_Op transa;
  Pad_Op pada;
  BLAS_Op transb;
  Pad_Op padb;
  BLAS_Op transc;
  Pad_Op padc;

  GEMM_Options_Pad() = default;
  GEMM_Options_Pad(BLAS_Op transa, Pad_Op pada, BLAS_Op transb, Pad_Op padb, BLAS_Op transc,
                   Pad_Op padc)
      : transa(transa), pada(pada), transb(transb), padb(padb), transc(transc), padc(padc) {}
  auto switches() { return std::tie(transa, transb, transc, pada, padb, padc); }
  auto switches() const { return std::tie(transa, transb, transc, pada, padb, padc); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(GEMM_Inputs<T>);
};

// Variant "[ta][tb][tc]/<tile>": the transposes plus the macro-tile shape of the GEMM
// kernel ("auto" first: the default variant is the plain call).  No counterpart in the
// reference: it is the kernel-variant axis a vendor BLAS hides, exposed for the planner to time.
struct GEMM_Options_Tile : Switch_Variant<GEMM_Options_Tile> {
  BLAS_Op transa, transb, transc;
  Tile_Op tile;

  GEMM_Options_Tile() = default;
  GEMM_Options_Tile(BLAS_Op transa, BLAS_Op transb, BLAS_Op transc, Tile_Op tile)
      : transa(transa), transb(transb), transc(transc), tile(tile) {}
  auto switches() { return std::tie(transa, transb, transc, tile); }
  auto switches() const { return std::tie(transa, transb, transc, tile); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(GEMM_Inputs<T>);
};

// Variant "[ta][tb][tc][pa][pb][pc]/<tile>/<tail>": the reference's transpose and pad switches
// (gemm.cpp:28-39) jointly with the kernel's own choices - macro-tile shape and what happens
// to the tiles of the last partial round - so that "pad to the tile and unpad" is timed
// against "masked edge" under every tile shape, not only the default one.  960 settings: meant
// to be explored under an Option_Filter (a pattern, or one learned from earlier timings).
struct GEMM_Options_Pad_Tile : Switch_Variant<GEMM_Options_Pad_Tile> {
  BLAS_Op transa, transb, transc;
  Pad_Op pada, padb, padc;
  Tile_Op tile;
  Tail_Op tail;

  GEMM_Options_Pad_Tile() = default;
  GEMM_Options_Pad_Tile(BLAS_Op transa, BLAS_Op transb, BLAS_Op transc, Pad_Op pada, Pad_Op padb,
                        Pad_Op padc, Tile_Op tile, Tail_Op tail)
      : transa(transa), transb(transb), transc(transc), pada(pada), padb(padb), padc(padc),
        tile(tile), tail(tail) {}
  auto switches() { return std::tie(transa, transb, transc, pada, padb, padc, tile, tail); }
  auto switches() const { return std::tie(transa, transb, transc, pada, padb, padc, tile, tail); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(GEMM_Inputs<T>);
};

// GEMM_Options whose tc also takes the letter X: the transposed result formed by the kernel
// itself in one launch (Fusable_Op, base_options.h).  Every kernel here takes its operands in
// either orientation, so that form is the plain call on C: "??X" builds the tree of "??N", needs
// no scratch, and is not enumerated beside it.  (The reference's tree can only express the
// transposition as a second pass, gemm.cpp:205-214.)
struct GEMM_Options_Fused : Switch_Variant<GEMM_Options_Fused> {
  BLAS_Op transa, transb;
  Fusable_Trans_Op transc;

  GEMM_Options_Fused() = default;
  GEMM_Options_Fused(BLAS_Op transa, BLAS_Op transb, Fusable_Trans_Op transc)
      : transa(transa), transb(transb), transc(transc) {}
  auto switches() { return std::tie(transa, transb, transc); }
  auto switches() const { return std::tie(transa, transb, transc); }

  template <typename T>
  std::unique_ptr<MatrixOp<T>> form_operation(GEMM_Inputs<T>);
};

namespace detail {
// Tiny gemm and geam calls in every op combination, so that first-launch costs (code object
// load, LDS attribute set-up) are paid before anything is timed (reference gemm.h:117-139).
template <typename T>
void warm_gemm_kernels(gpu::blasHandle_t handle);
}  // namespace detail

template <typename T>
using GEMM_Executor =
    Warmed_Executor<GEMM_Inputs<T>, GEMM_Key, GEMM_Options, &detail::warm_gemm_kernels<T>>;
template <typename T>
using GEMM_Executor_Pad =
    Warmed_Executor<GEMM_Inputs<T>, GEMM_Key, GEMM_Options_Pad, &detail::warm_gemm_kernels<T>>;
template <typename T>
using GEMM_Executor_Fused =
    Warmed_Executor<GEMM_Inputs<T>, GEMM_Key, GEMM_Options_Fused, &detail::warm_gemm_kernels<T>>;
template <typename T>
using GEMM_Executor_Tile =
    Warmed_Executor<GEMM_Inputs<T>, GEMM_Key, GEMM_Options_Tile, &detail::warm_gemm_kernels<T>>;
template <typename T>
using GEMM_Executor_Pad_Tile = Warmed_Executor<GEMM_Inputs<T>, GEMM_Key, GEMM_Options_Pad_Tile,
                                               &detail::warm_gemm_kernels<T>>;

}  // namespace rtat
