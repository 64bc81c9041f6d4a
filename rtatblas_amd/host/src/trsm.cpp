#include "trsm.h"

namespace rtat {

std::string TRSM_Key::spell(BLAS_Side side, BLAS_Fill_Mode uplo, BLAS_Operation trans,
                            BLAS_Diag diag, int m, int n) {
  return std::string(side) + "," + std::string(uplo) + "," + std::string(trans) + "," +
         std::string(diag) + "," + std::to_string(m) + "," + std::to_string(n);
}

// Reference trsm.cpp:72-111.  transpose_A: A^T in scratch; the stored triangle and the op
// flag both flip.  swap_side: op(A) X = alpha B  <=>  X^T op(A)^T = alpha B^T, so B^T goes to
// scratch, is solved there on the other side with the op flag flipped, and is written back
// transposed over B (beta = 0: B's old contents are not read again).
namespace {
template <typename T>
std::unique_ptr<MatrixOp<T>> build_trsm_tree(TRSM_Inputs<T> params, bool swap_side,
                                             bool transpose_A, int kernel = RTAT_GEMM_AUTO);
}

template <typename T>
std::unique_ptr<MatrixOp<T>> TRSM_Options::form_operation(TRSM_Inputs<T> params) {
  return build_trsm_tree<T>(params, swap_side, transpose_A);
}

// "X?" is the plain solve on B: see TRSM_Options_Fused.
template <typename T>
std::unique_ptr<MatrixOp<T>> TRSM_Options_Fused::form_operation(TRSM_Inputs<T> params) {
  return build_trsm_tree<T>(params, swap_side == Fusable_Bool_Op::ON, transpose_A);
}

// The reference's switches with the kernel options handed to the TRSM node.
template <typename T>
std::unique_ptr<MatrixOp<T>> TRSM_Options_Tile::form_operation(TRSM_Inputs<T> params) {
  return build_trsm_tree<T>(params, swap_side, transpose_A,
                            RTAT_KERNEL_OPTIONS(tile.id, tail.id, panel.id));
}

namespace {
template <typename T>
std::unique_ptr<MatrixOp<T>> build_trsm_tree(TRSM_Inputs<T> params, bool swap_side,
                                             bool transpose_A, int kernel) {
  std::unique_ptr<MatrixOp<T>> A = std::make_unique<NoOp<T>>(params.A);
  std::unique_ptr<MatrixOp<T>> B = std::make_unique<NoOp<T>>(params.B);
  bool left = params.side == gpu::BLAS_SIDE_LEFT;
  bool lower = params.uplo == gpu::BLAS_FILL_MODE_LOWER;
  bool trans = params.trans == gpu::BLAS_OP_T;
  const bool unit = params.diag == gpu::BLAS_DIAG_UNIT;

  if (transpose_A) {
    trans = !trans;
    lower = !lower;
    A = std::make_unique<MatrixMove<T>>(std::move(A), T(1), true, 1);
  }
  if (swap_side) {
    trans = !trans;
    left = !left;
    std::unique_ptr<MatrixOp<T>> Bt = std::make_unique<MatrixMove<T>>(std::move(B), T(1), true, 1);
    std::unique_ptr<MatrixOp<T>> S = std::make_unique<MatrixTrsAlloc<T>>(
        std::move(A), std::move(Bt), left, lower, trans, unit, params.alpha, 1, kernel);
    std::unique_ptr<MatrixOp<T>> target = std::make_unique<NoOp<T>>(params.B);
    return std::make_unique<MatrixAccumulate<T>>(std::move(S), std::move(target), T(1), T(0),
                                                 true);
  }
  return std::make_unique<MatrixTrs<T>>(std::move(A), std::move(B), left, lower, trans, unit,
                                        params.alpha, kernel);
}
}  // namespace

namespace detail {
// Reference trsm.h:87-113: a small solve + geam for every side / uplo / trans combination.
template <typename T>
void warm_trsm_kernels(gpu::blasHandle_t handle) {
  constexpr size_t n = 128;
  ManagedWorkspace mem(3 * n * n * sizeof(T));
  Workspace rest = mem;
  Matrix<T> A(rest.peel<T>(n * n), n, n, n), B(rest.peel<T>(n * n), n, n, n),
      D(rest.peel<T>(n * n), n, n, n);
  gpuAssert(gpu::Memset((T*)mem, 0, 3 * n * n * sizeof(T)));
  // A = 0 with a unit diagonal assumed: the solves are well defined and trivial.
  for (bool left : {false, true})
    for (bool lower : {false, true})
      for (bool trans : {false, true}) {
        blas_check(gpuTtrsm<T>(handle, left, lower, trans, true, A, B, T(1)), "trsm warm-up");
        blas_check(gpuTgeam<T>(handle, true, false, A, B, D, T(1), T(0)), "geam warm-up");
      }
  gpuAssert(gpu::DeviceSynchronize());
}
template void warm_trsm_kernels<double>(gpu::blasHandle_t);
template void warm_trsm_kernels<float>(gpu::blasHandle_t);
}  // namespace detail

template std::unique_ptr<MatrixOp<double>> TRSM_Options::form_operation(TRSM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> TRSM_Options::form_operation(TRSM_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> TRSM_Options_Fused::form_operation(TRSM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> TRSM_Options_Fused::form_operation(TRSM_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> TRSM_Options_Tile::form_operation(TRSM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> TRSM_Options_Tile::form_operation(TRSM_Inputs<float>);

}  // namespace rtat
