#include "gemm.h"

namespace rtat {

// ---- kernel-option switches: every value the library names, "auto" (id 0) first ----------------
namespace {
template <class Op>
std::vector<Op> every_named_value(const char* (*name)(int)) {
  std::vector<Op> all;
  for (int v = 0; name(v) != nullptr; ++v) all.push_back(Op(v));
  return all;
}
}  // namespace
std::vector<Tile_Op> Tile_Op::enumerate() { return every_named_value<Tile_Op>(rtat_gemm_variant_name); }
std::vector<Tail_Op> Tail_Op::enumerate() { return every_named_value<Tail_Op>(rtat_tail_mode_name); }
std::vector<Panel_Op> Panel_Op::enumerate() { return every_named_value<Panel_Op>(rtat_trsm_panel_name); }

// ---- GEMM_Key ----------------------------------------------------------------------------------
std::string GEMM_Key::spell(BLAS_Operation ta, BLAS_Operation tb, int m, int k, int n) {
  return std::string(ta) + "," + std::string(tb) + ",," + std::to_string(m) + "," +
         std::to_string(k) + "," + std::to_string(n);
}

namespace {

template <typename T>
using Node = std::unique_ptr<MatrixOp<T>>;

// The tree every GEMM variant family builds (reference gemm.cpp:75-134 and :183-221):
//   * transposing an input = materialise op^T in scratch and flip the flag handed to the kernel;
//   * padding an input     = copy it to a leading dimension that is a multiple of 32 elements;
//   * transposing C        = form (alpha op(A) op(B))^T = alpha op(B)^T op(A)^T in scratch, then
//                            C = S^T + beta C;
//   * padding C            = form the product in padded scratch, then C = S + beta C.
template <typename T>
Node<T> build_gemm_tree(GEMM_Inputs<T> in, bool ta, bool tb, bool tc, bool pa, bool pb, bool pc,
                        int tile) {
  constexpr size_t PAD = 32;
  Node<T> A = std::make_unique<NoOp<T>>(in.A);
  Node<T> B = std::make_unique<NoOp<T>>(in.B);
  Node<T> C = std::make_unique<NoOp<T>>(in.C);
  bool a_trans = in.transa == gpu::BLAS_OP_T, b_trans = in.transb == gpu::BLAS_OP_T;

  if (ta) a_trans = !a_trans;
  if (ta || pa) A = std::make_unique<MatrixMove<T>>(std::move(A), T(1), ta, pa ? PAD : 1);
  if (tb) b_trans = !b_trans;
  if (tb || pb) B = std::make_unique<MatrixMove<T>>(std::move(B), T(1), tb, pb ? PAD : 1);

  if (tc) {
    Node<T> S = std::make_unique<MatrixMultAlloc<T>>(std::move(B), std::move(A), !b_trans,
                                                     !a_trans, in.alpha, pc ? PAD : 1, tile);
    return std::make_unique<MatrixAccumulate<T>>(std::move(S), std::move(C), T(1), in.beta, true);
  }
  if (pc) {
    Node<T> S = std::make_unique<MatrixMultAlloc<T>>(std::move(A), std::move(B), a_trans, b_trans,
                                                     in.alpha, PAD, tile);
    return std::make_unique<MatrixAccumulate<T>>(std::move(S), std::move(C), T(1), in.beta, false);
  }
  return std::make_unique<MatrixMult<T>>(std::move(A), std::move(B), std::move(C), a_trans,
                                         b_trans, in.alpha, in.beta, tile);
}

}  // namespace

// ---- the variant families: each hands its switches to the one tree builder --------------------
template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, false, false, false, RTAT_GEMM_AUTO);
}

template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options_Pad::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, pada == Pad_Op::PAD, padb == Pad_Op::PAD,
                            padc == Pad_Op::PAD, RTAT_GEMM_AUTO);
}

// "??X": (alpha op(B)^T op(A)^T)^T + beta C is alpha op(A) op(B) + beta C with the operand
// roles as the caller gave them; the kernel takes either orientation of either operand, so
// the tree's scratch product and transposing pass collapse into the one multiply on C.
template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options_Fused::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == Fusable_Trans_Op::ON, false, false, false, RTAT_GEMM_AUTO);
}

template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options_Tile::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, false, false, false, tile.id);
}

template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options_Pad_Tile::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, pada == Pad_Op::PAD, padb == Pad_Op::PAD,
                            padc == Pad_Op::PAD,
                            RTAT_KERNEL_OPTIONS(tile.id, tail.id, RTAT_PANEL_AUTO));
}

// ---- warm-up ---------------------------------------------------------------------------------------
namespace detail {
template <typename T>
void warm_gemm_kernels(gpu::blasHandle_t handle) {
  constexpr size_t n = 8;
  ManagedWorkspace mem(3 * n * n * sizeof(T));
  Workspace rest = mem;
  Matrix<T> A(rest.peel<T>(n * n), n, n, n), B(rest.peel<T>(n * n), n, n, n),
      C(rest.peel<T>(n * n), n, n, n);
  gpuAssert(gpu::Memset((T*)mem, 0, 3 * n * n * sizeof(T)));
  for (bool ta : {false, true})
    for (bool tb : {false, true}) {
      blas_check(gpuTgemm<T>(handle, ta, tb, A, B, C, T(1), T(0)), "gemm warm-up");
      blas_check(gpuTgeam<T>(handle, ta, false, A, B, C, T(1), T(0)), "geam warm-up");
    }
  gpuAssert(gpu::DeviceSynchronize());
}
template void warm_gemm_kernels<double>(gpu::blasHandle_t);
template void warm_gemm_kernels<float>(gpu::blasHandle_t);
}  // namespace detail

template std::unique_ptr<MatrixOp<double>> GEMM_Options::form_operation(GEMM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> GEMM_Options::form_operation(GEMM_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> GEMM_Options_Pad::form_operation(GEMM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> GEMM_Options_Pad::form_operation(GEMM_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> GEMM_Options_Fused::form_operation(GEMM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> GEMM_Options_Fused::form_operation(GEMM_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> GEMM_Options_Tile::form_operation(GEMM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> GEMM_Options_Tile::form_operation(GEMM_Inputs<float>);
template std::unique_ptr<MatrixOp<double>> GEMM_Options_Pad_Tile::form_operation(GEMM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> GEMM_Options_Pad_Tile::form_operation(GEMM_Inputs<float>);

}  // namespace rtat
