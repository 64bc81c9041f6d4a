#include "syrk.h"

namespace rtat {

std::string SYRK_Key::spell(BLAS_Fill_Mode uplo, BLAS_Operation trans, int n, int k) {
  return std::string(uplo) + "," + std::string(trans) + "," + std::to_string(n) + "," +
         std::to_string(k);
}

// Reference syrk.cpp:71-104.  transpose_A: A^T in scratch, trans flag flipped.  transpose_C:
// the opposite triangle of a zeroed n x n scratch S gets alpha op(A) op(A)^T, then
// C = S^T + beta C over the WHOLE of C — so, as in the reference, the triangle the caller did
// not ask for comes back scaled by beta rather than untouched.
namespace {
template <typename T>
std::unique_ptr<MatrixOp<T>> build_syrk_tree(SYRK_Inputs<T> params, bool transpose_A,
                                             bool transpose_C, int kernel = RTAT_GEMM_AUTO);
}

template <typename T>
std::unique_ptr<MatrixOp<T>> SYRK_Options::form_operation(SYRK_Inputs<T> params) {
  return build_syrk_tree<T>(params, transpose_A, transpose_C);
}

// "?X" is the plain SYRK on C: see SYRK_Options_Fused.
template <typename T>
std::unique_ptr<MatrixOp<T>> SYRK_Options_Fused::form_operation(SYRK_Inputs<T> params) {
  return build_syrk_tree<T>(params, transpose_A, transpose_C == Fusable_Bool_Op::ON);
}

// The reference's switches with the kernel options handed to the SYRK node.
template <typename T>
std::unique_ptr<MatrixOp<T>> SYRK_Options_Tile::form_operation(SYRK_Inputs<T> params) {
  return build_syrk_tree<T>(params, transpose_A, transpose_C,
                            RTAT_KERNEL_OPTIONS(tile.id, tail.id, RTAT_PANEL_AUTO));
}

namespace {
template <typename T>
std::unique_ptr<MatrixOp<T>> build_syrk_tree(SYRK_Inputs<T> params, bool transpose_A,
                                             bool transpose_C, int kernel) {
  std::unique_ptr<MatrixOp<T>> A = std::make_unique<NoOp<T>>(params.A);
  std::unique_ptr<MatrixOp<T>> C = std::make_unique<NoOp<T>>(params.C);
  bool trans = params.trans == gpu::BLAS_OP_T;
  bool lower = params.uplo == gpu::BLAS_FILL_MODE_LOWER;

  if (transpose_A) {
    trans = !trans;
    A = std::make_unique<MatrixMove<T>>(std::move(A), T(1), true, 1);
  }
  if (transpose_C) {
    std::unique_ptr<MatrixOp<T>> S =
        std::make_unique<MatrixSyrkAlloc<T>>(std::move(A), !lower, trans, params.alpha, 1, kernel);
    return std::make_unique<MatrixAccumulate<T>>(std::move(S), std::move(C), T(1), params.beta,
                                                 true);
  }
  return std::make_unique<MatrixSyrk<T>>(std::move(A), std::move(C), lower, trans, params.alpha,
                                         params.beta, kernel);
}
}  // namespace

namespace detail {
// Reference syrk.h:82-115: small syrk + geam in every uplo / trans combination.
template <typename T>
void warm_syrk_kernels(gpu::blasHandle_t handle) {
  constexpr size_t n = 64;
  ManagedWorkspace mem(3 * n * n * sizeof(T));
  Workspace rest = mem;
  Matrix<T> A(rest.peel<T>(n * n), n, n, n), C(rest.peel<T>(n * n), n, n, n),
      D(rest.peel<T>(n * n), n, n, n);
  gpuAssert(gpu::Memset((T*)mem, 0, 3 * n * n * sizeof(T)));
  for (bool lower : {false, true})
    for (bool trans : {false, true}) {
      blas_check(gpuTsyrk<T>(handle, lower, trans, A, C, T(1), T(0)), "syrk warm-up");
      blas_check(gpuTgeam<T>(handle, true, false, A, C, D, T(1), T(0)), "geam warm-up");
    }
  gpuAssert(gpu::DeviceSynchronize());
}
template void warm_syrk_kernels<double>(gpu::blasHandle_t);
template void warm_syrk_kernels<float>(gpu::blasHandle_t);
}  // namespace detail

template std::unique_ptr<MatrixOp<double>> SYRK_Options::form_operation(SYRK_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> SYRK_Options::form_operation(SYRK_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> SYRK_Options_Fused::form_operation(SYRK_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> SYRK_Options_Fused::form_operation(SYRK_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> SYRK_Options_Tile::form_operation(SYRK_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> SYRK_Options_Tile::form_operation(SYRK_Inputs<float>);

}  // namespace rtat
