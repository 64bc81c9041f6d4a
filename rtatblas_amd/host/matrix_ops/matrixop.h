// Lazy matrix-op tree: a description of a small matrix computation that is made concrete by
// handing it output space, scratch space and an execution context.
//
// Mirrors the reference's src/matrix_ops/matrixop.h — same node classes, constructor
// arguments, dims()/output_space_req()/workspace_req() rules and execute() protocol — so the
// variant builders in src/methods and user code compile against it unchanged.  What differs:
// the four shims call the gfx950 kernels of rtat_native.h instead of a vendor BLAS, every
// status is checked (a failed launch throws), shape errors throw std::invalid_argument
// instead of terminating, the GEMM-family nodes carry an optional kernel-variant id, and a
// multiply whose two inputs are both plain moves of existing matrices issues them as one
// launch.
#pragma once
#include <gpu-api.h>

#include <memory>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "matrix.h"

namespace rtat {

template <typename T>
inline constexpr bool is_blas_scalar = std::is_same_v<T, double> || std::is_same_v<T, float>;

inline gpu::blasOperation_t op_of(bool trans) { return trans ? gpu::BLAS_OP_T : gpu::BLAS_OP_N; }
inline gpu::blasFillMode_t fill_of(bool lower) {
  return lower ? gpu::BLAS_FILL_MODE_LOWER : gpu::BLAS_FILL_MODE_UPPER;
}

// ---- the four BLAS shims (reference matrixop.h:15-140) -----------------------------------
// Sizes are derived from the Matrix views exactly as the reference does: m, n from C and k
// from A for gemm (:20-22); n from C and k from A for syrk (:53-54); m, n from B for trsm
// (:84-85) and — note — from B, not C, for geam (:121).

template <typename T>
inline gpu::blasStatus_t gpuTgemm(gpu::blasHandle_t handle, bool transa, bool transb, Matrix<T> A,
                                  Matrix<T> B, Matrix<T> C, const T alpha, const T beta,
                                  int variant = RTAT_GEMM_AUTO) {
  static_assert(is_blas_scalar<T>, "GEMM is only double and float");
  const int m = (int)C.dims().m, n = (int)C.dims().n;
  const int k = (int)(transa ? A.dims().m : A.dims().n);
  if constexpr (std::is_same_v<T, double>)
    return gpu::blasDgemmEx(handle, op_of(transa), op_of(transb), m, n, k, &alpha, A.ptr(),
                            (int)A.dims().ld, B.ptr(), (int)B.dims().ld, &beta, C.ptr(),
                            (int)C.dims().ld, variant);
  else
    return gpu::blasSgemmEx(handle, op_of(transa), op_of(transb), m, n, k, &alpha, A.ptr(),
                            (int)A.dims().ld, B.ptr(), (int)B.dims().ld, &beta, C.ptr(),
                            (int)C.dims().ld, variant);
}

template <typename T>
inline gpu::blasStatus_t gpuTsyrk(gpu::blasHandle_t handle, bool lower, bool trans, Matrix<T> A,
                                  Matrix<T> C, const T alpha, const T beta,
                                  int variant = RTAT_GEMM_AUTO) {
  static_assert(is_blas_scalar<T>, "SYRK is only double and float");
  const int n = (int)C.dims().n;
  const int k = (int)(trans ? A.dims().m : A.dims().n);
  if constexpr (std::is_same_v<T, double>)
    return gpu::blasDsyrkEx(handle, fill_of(lower), op_of(trans), n, k, &alpha, A.ptr(),
                            (int)A.dims().ld, &beta, C.ptr(), (int)C.dims().ld, variant);
  else
    return gpu::blasSsyrkEx(handle, fill_of(lower), op_of(trans), n, k, &alpha, A.ptr(),
                            (int)A.dims().ld, &beta, C.ptr(), (int)C.dims().ld, variant);
}

template <typename T>
inline gpu::blasStatus_t gpuTtrsm(gpu::blasHandle_t handle, bool side_left, bool lower, bool trans,
                                  bool unit_diag, Matrix<T> A, Matrix<T> B, const T alpha,
                                  int variant = RTAT_GEMM_AUTO) {
  static_assert(is_blas_scalar<T>, "TRSM is only double and float");
  const int m = (int)B.dims().m, n = (int)B.dims().n;
  const auto side = side_left ? gpu::BLAS_SIDE_LEFT : gpu::BLAS_SIDE_RIGHT;
  const auto diag = unit_diag ? gpu::BLAS_DIAG_UNIT : gpu::BLAS_DIAG_NON_UNIT;
  if constexpr (std::is_same_v<T, double>)
    return gpu::blasDtrsmEx(handle, side, fill_of(lower), op_of(trans), diag, m, n, &alpha,
                            A.ptr(), (int)A.dims().ld, B.ptr(), (int)B.dims().ld, variant);
  else
    return gpu::blasStrsmEx(handle, side, fill_of(lower), op_of(trans), diag, m, n, &alpha,
                            A.ptr(), (int)A.dims().ld, B.ptr(), (int)B.dims().ld, variant);
}

template <typename T>
inline gpu::blasStatus_t gpuTgeam(gpu::blasHandle_t handle, bool transa, bool transb, Matrix<T> A,
                                  Matrix<T> B, Matrix<T> C, const T alpha, const T beta) {
  static_assert(is_blas_scalar<T>, "GEAM is only double and float");
  const int m = (int)B.dims().m, n = (int)B.dims().n;
  if constexpr (std::is_same_v<T, double>)
    return gpu::blasDgeam(handle, op_of(transa), op_of(transb), m, n, &alpha, A.ptr(),
                          (int)A.dims().ld, &beta, B.ptr(), (int)B.dims().ld, C.ptr(),
                          (int)C.dims().ld);
  else
    return gpu::blasSgeam(handle, op_of(transa), op_of(transb), m, n, &alpha, A.ptr(),
                          (int)A.dims().ld, &beta, B.ptr(), (int)B.dims().ld, C.ptr(),
                          (int)C.dims().ld);
}

// B_i = op_i(A_i) for two pairs in one launch (no counterpart in the reference): the fused
// form of two MatrixMove nodes with alpha = 1.  Sizes come from the B views, as in gpuTgeam.
template <typename T>
inline gpu::blasStatus_t gpuTmovePair(gpu::blasHandle_t handle, bool trans0, Matrix<T> A0,
                                      Matrix<T> B0, bool trans1, Matrix<T> A1, Matrix<T> B1) {
  static_assert(is_blas_scalar<T>, "moves are only double and float");
  gpu::blasMove_t jobs[2] = {
      {op_of(trans0), (int)B0.dims().m, (int)B0.dims().n, A0.ptr(), (int)A0.dims().ld, B0.ptr(),
       (int)B0.dims().ld},
      {op_of(trans1), (int)B1.dims().m, (int)B1.dims().n, A1.ptr(), (int)A1.dims().ld, B1.ptr(),
       (int)B1.dims().ld}};
  if constexpr (std::is_same_v<T, double>) return gpu::blasDmovePair(handle, &jobs[0], &jobs[1]);
  else return gpu::blasSmovePair(handle, &jobs[0], &jobs[1]);
}

// ---- node protocol (reference matrixop.h:142-215) -----------------------------------------
template <typename T>
class MatrixOp {
 public:
  using Ptr = std::unique_ptr<MatrixOp<T>>;

  MatrixOp(const MatrixOp&) = delete;
  MatrixOp(MatrixOp&&) = default;
  MatrixOp& operator=(MatrixOp&&) = default;
  explicit MatrixOp(std::vector<Ptr> operands, int output_operand = -1)
      : operands(std::move(operands)), output_operand(output_operand) {}
  virtual ~MatrixOp() = default;

  // Compute the result.  `out_space` receives it when the node produces a fresh matrix
  // (output_space_req() > 0); `scratch_space` serves the operands.
  virtual Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                            Workspace scratch_space) = 0;
  // Elements of T the node's own result needs in out_space (0: it writes into an operand).
  virtual size_t output_space_req() const = 0;
  virtual MatrixDims dims() const = 0;

  // Elements of T needed in total: the own output plus the high-water mark, walking the
  // operands in order, of (outputs of the operands so far that do not land in out_space) +
  // (scratch of the operand being computed).  (reference :172-185)
  size_t workspace_req() const {
    size_t held = 0, peak = 0;
    for (int i = 0; i < (int)operands.size(); ++i) {
      if (i != output_operand) held += operands[i]->output_space_req();
      peak = std::max(peak, held + operands[i]->scratch_space_req());
    }
    return output_space_req() + peak;
  }
  size_t scratch_space_req() const { return workspace_req() - output_space_req(); }
  size_t workspace_req_bytes() const { return sizeof(T) * workspace_req(); }
  size_t scratch_space_req_bytes() const { return sizeof(T) * scratch_space_req(); }

  // Evaluate the operands in order.  The output operand is computed straight into
  // out_space; every other operand's result is peeled off the front of the scratch, and the
  // operand itself works in what is left behind it.  (reference :192-210)
  std::vector<Matrix<T>> compute_operands(gpu::blasHandle_t handle, Workspace out_space,
                                          Workspace scratch_space) {
    std::vector<Matrix<T>> results;
    results.reserve(operands.size());
    for (int i = 0; i < (int)operands.size(); ++i) {
      Workspace target = (i == output_operand)
                             ? out_space
                             : scratch_space.template peel<T>(operands[i]->output_space_req());
      results.push_back(operands[i]->execute(handle, target, scratch_space));
    }
    return results;
  }
  std::vector<Matrix<T>> compute_operands(gpu::blasHandle_t handle, Workspace scratch_space) {
    return compute_operands(handle, Workspace(), scratch_space);
  }

 protected:
  void require_space(Workspace& out_space, Workspace& scratch_space, const char* who) const {
    if (out_space.size<T>() < output_space_req() || scratch_space.size<T>() < scratch_space_req())
      throw std::runtime_error(std::string(who) + ": not enough space");
  }
  std::vector<Ptr> operands;
  int output_operand = -1;
};

// An existing matrix (reference :217-229).
template <typename T>
class NoOp : public MatrixOp<T> {
  Matrix<T> A;

 public:
  NoOp(Matrix<T> A) : MatrixOp<T>({}), A(A) {}
  Matrix<T> execute(gpu::blasHandle_t, Workspace, Workspace) override { return A; }
  size_t output_space_req() const override { return 0; }
  MatrixDims dims() const override { return A.dims(); }
};

// Uninitialised scratch of a given shape (reference :231-254).
template <typename T>
class ScratchMatrix : public MatrixOp<T> {
  MatrixDims shape;

 public:
  ScratchMatrix(MatrixDims dims) : MatrixOp<T>({}), shape(dims) {}
  ScratchMatrix(size_t m, size_t n, size_t ld) : ScratchMatrix(MatrixDims(m, n, ld)) {}
  // Shaped like `op`'s result with the leading dimension padded to a multiple of `pad`.
  ScratchMatrix(std::unique_ptr<MatrixOp<T>>& op, int pad)
      : ScratchMatrix(op->dims().repadded(pad)) {}
  size_t output_space_req() const override { return shape.footprint(); }
  MatrixDims dims() const override { return shape; }
  Matrix<T> execute(gpu::blasHandle_t, Workspace out_space, Workspace) override {
    return Matrix<T>(out_space, shape);
  }
};

// B = alpha op(A) + beta B, in place on operand B (reference :256-305): un-pad, transpose
// back, accumulate into the caller's matrix.
template <typename T>
class MatrixAccumulate : public MatrixOp<T> {
  T alpha, beta;
  bool transpose;

 public:
  MatrixAccumulate(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Bop, T alpha,
                   T beta, bool transpose)
      : MatrixOp<T>({}, 1), alpha(alpha), beta(beta), transpose(transpose) {
    const MatrixDims a = Aop->dims(), b = Bop->dims();
    const bool fits = transpose ? (a.m == b.n && a.n == b.m) : (a.m == b.m && a.n == b.n);
    if (!fits)
      throw std::invalid_argument("Bad matrix accumulate, Adims=" + std::to_string(a.m) + "," +
                                  std::to_string(a.n) + " Bdims=" + std::to_string(b.m) + "," +
                                  std::to_string(b.n) + (transpose ? " trans" : " notrans"));
    this->operands.push_back(std::move(Aop));
    this->operands.push_back(std::move(Bop));
  }
  size_t output_space_req() const override { return 0; }
  MatrixDims dims() const override { return this->operands[1]->dims(); }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    this->require_space(out_space, scratch_space, "MatrixAccumulate");
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    blas_check(gpuTgeam<T>(handle, transpose, false, mats[0], mats[1], mats[1], alpha, beta),
               "geam (MatrixAccumulate)");
    return mats[1];
  }
};

// Fresh B = alpha op(A), leading dimension padded to a multiple of `pad` (reference
// :307-344): copy, transpose, re-stride.  Rows m..ld-1 of B are left as they were.
template <typename T>
class MatrixMove : public MatrixOp<T> {
  T alpha;
  bool transpose;
  size_t pad;

 public:
  MatrixMove(std::unique_ptr<MatrixOp<T>> Aop, T alpha, bool transpose, size_t pad)
      : MatrixOp<T>({}), alpha(alpha), transpose(transpose), pad(pad) {
    if (pad == 0) throw std::invalid_argument("MatrixMove: pad must be positive");
    this->operands.push_back(std::move(Aop));
  }
  size_t output_space_req() const override { return dims().footprint(); }
  MatrixDims dims() const override {
    const MatrixDims a = this->operands[0]->dims();
    return transpose ? a.transposed(pad) : a.repadded(pad);
  }
  // A plain move of an existing matrix (alpha = 1, the source needs no computing): such a
  // node's whole work is one copy or transpose, which a parent with two of them can issue as
  // one launch (gpuTmovePair).  The source matrix, when that holds.
  bool moves_existing_matrix() const {
    return alpha == T(1) && this->operands[0]->output_space_req() == 0 &&
           this->operands[0]->scratch_space_req() == 0 &&
           dynamic_cast<const NoOp<T>*>(this->operands[0].get()) != nullptr;
  }
  Matrix<T> source(gpu::blasHandle_t handle) {
    return this->operands[0]->execute(handle, Workspace(), Workspace());
  }
  bool transposes() const { return transpose; }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    this->require_space(out_space, scratch_space, "MatrixMove");
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    Matrix<T> B(out_space, dims());
    blas_check(gpuTgeam<T>(handle, transpose, false, mats[0], B, B, alpha, T(0)),
               "geam (MatrixMove)");
    return B;
  }
};

namespace detail {
// Operands 0 and 1 of a multiply, evaluated as compute_operands would (results peeled off the
// front of the scratch in operand order), except that two plain moves of existing matrices go
// out as ONE launch instead of two.  Returns false, touching nothing, when the operands are
// not such a pair.
template <typename T>
inline bool compute_move_pair(std::vector<std::unique_ptr<MatrixOp<T>>>& operands,
                              gpu::blasHandle_t handle, Workspace& scratch_space,
                              std::vector<Matrix<T>>& results) {
  auto* first = dynamic_cast<MatrixMove<T>*>(operands[0].get());
  auto* second = dynamic_cast<MatrixMove<T>*>(operands[1].get());
  if (first == nullptr || second == nullptr || !first->moves_existing_matrix() ||
      !second->moves_existing_matrix())
    return false;
  if (scratch_space.size<T>() < first->output_space_req() + second->output_space_req())
    throw std::runtime_error("MatrixMove pair: not enough space");
  Matrix<T> B0(scratch_space.template peel<T>(first->output_space_req()), first->dims());
  Matrix<T> B1(scratch_space.template peel<T>(second->output_space_req()), second->dims());
  blas_check(gpuTmovePair<T>(handle, first->transposes(), first->source(handle), B0,
                             second->transposes(), second->source(handle), B1),
             "move pair (MatrixMove x 2)");
  results.push_back(B0);
  results.push_back(B1);
  return true;
}

inline void check_inner(size_t ka, size_t kb) {
  if (ka != kb)
    throw std::invalid_argument("Bad matrix mult, kA=" + std::to_string(ka) +
                                " kB=" + std::to_string(kb));
}
}  // namespace detail

// C = alpha op(A) op(B) + beta C into operand C (reference :347-395).
template <typename T>
class MatrixMult : public MatrixOp<T> {
 protected:
  bool transa, transb;
  T alpha, beta;
  int variant;

 public:
  MatrixMult(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Bop,
             std::unique_ptr<MatrixOp<T>> Cop, bool transa, bool transb, T alpha, T beta,
             int variant = RTAT_GEMM_AUTO)
      : MatrixOp<T>({}, 2), transa(transa), transb(transb), alpha(alpha), beta(beta),
        variant(variant) {
    const MatrixDims a = Aop->dims(), b = Bop->dims(), c = Cop->dims();
    detail::check_inner(transa ? a.m : a.n, transb ? b.n : b.m);
    if ((transa ? a.n : a.m) != c.m || (transb ? b.m : b.n) != c.n)
      throw std::invalid_argument("Bad matrix mult, C is " + std::to_string(c.m) + "x" +
                                  std::to_string(c.n));
    this->operands.push_back(std::move(Aop));
    this->operands.push_back(std::move(Bop));
    this->operands.push_back(std::move(Cop));
  }
  MatrixDims dims() const override { return this->operands[2]->dims(); }
  size_t output_space_req() const override { return 0; }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    std::vector<Matrix<T>> mats;
    if (detail::compute_move_pair<T>(this->operands, handle, scratch_space, mats))
      mats.push_back(this->operands[2]->execute(handle, out_space, scratch_space));
    else
      mats = this->compute_operands(handle, out_space, scratch_space);
    blas_check(gpuTgemm<T>(handle, transa, transb, mats[0], mats[1], mats[2], alpha, beta, variant),
               "gemm (MatrixMult)");
    return mats[2];
  }
};

// Fresh C = alpha op(A) op(B), leading dimension padded (reference :397-440).
template <typename T>
class MatrixMultAlloc : public MatrixOp<T> {
  bool transa, transb;
  T alpha;
  size_t pad;
  int variant;

 public:
  MatrixMultAlloc(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Bop, bool transa,
                  bool transb, T alpha, size_t pad, int variant = RTAT_GEMM_AUTO)
      : MatrixOp<T>({}), transa(transa), transb(transb), alpha(alpha), pad(pad),
        variant(variant) {
    const MatrixDims a = Aop->dims(), b = Bop->dims();
    detail::check_inner(transa ? a.m : a.n, transb ? b.n : b.m);
    this->operands.push_back(std::move(Aop));
    this->operands.push_back(std::move(Bop));
  }
  MatrixDims dims() const override {
    const MatrixDims a = this->operands[0]->dims(), b = this->operands[1]->dims();
    const size_t m = transa ? a.n : a.m, n = transb ? b.m : b.n;
    return MatrixDims(m, n, padded_ld(m, pad));
  }
  size_t output_space_req() const override { return dims().footprint(); }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    this->require_space(out_space, scratch_space, "MatrixMultAlloc");
    std::vector<Matrix<T>> mats;
    if (!detail::compute_move_pair<T>(this->operands, handle, scratch_space, mats))
      mats = this->compute_operands(handle, out_space, scratch_space);
    Matrix<T> C(out_space, dims());
    blas_check(gpuTgemm<T>(handle, transa, transb, mats[0], mats[1], C, alpha, T(0), variant),
               "gemm (MatrixMultAlloc)");
    return C;
  }
};

namespace detail {
inline void check_trs(const MatrixDims& a, const MatrixDims& b, bool side_left) {
  if (a.m != a.n || (side_left ? b.m : b.n) != a.m)
    throw std::invalid_argument("Bad matrix trs, A is " + std::to_string(a.m) + "x" +
                                std::to_string(a.n) + ", B is " + std::to_string(b.m) + "x" +
                                std::to_string(b.n) + (side_left ? " LEFT" : " RIGHT"));
}
}  // namespace detail

// Triangular solve in place on operand B (reference :442-486).
template <typename T>
class MatrixTrs : public MatrixOp<T> {
 protected:
  bool side_left, lower, trans, unit_diag;
  T alpha;
  int variant;

 public:
  MatrixTrs(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Bop, bool side_left,
            bool lower, bool trans, bool unit_diag, T alpha, int variant = RTAT_GEMM_AUTO)
      : MatrixOp<T>({}, 1), side_left(side_left), lower(lower), trans(trans),
        unit_diag(unit_diag), alpha(alpha), variant(variant) {
    detail::check_trs(Aop->dims(), Bop->dims(), side_left);
    this->operands.push_back(std::move(Aop));
    this->operands.push_back(std::move(Bop));
  }
  MatrixDims dims() const override { return this->operands[1]->dims(); }
  size_t output_space_req() const override { return 0; }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    blas_check(gpuTtrsm<T>(handle, side_left, lower, trans, unit_diag, mats[0], mats[1], alpha,
                           variant),
               "trsm (MatrixTrs)");
    return mats[1];
  }
};

// Triangular solve on a fresh copy: operand B is computed into this node's out_space and
// solved there (reference :488-534).
template <typename T>
class MatrixTrsAlloc : public MatrixOp<T> {
 protected:
  bool side_left, lower, trans, unit_diag;
  T alpha;
  size_t pad;
  int variant;

 public:
  MatrixTrsAlloc(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Bop,
                 bool side_left, bool lower, bool trans, bool unit_diag, T alpha, size_t pad = 1,
                 int variant = RTAT_GEMM_AUTO)
      : MatrixOp<T>({}, 1), side_left(side_left), lower(lower), trans(trans),
        unit_diag(unit_diag), alpha(alpha), pad(pad), variant(variant) {
    detail::check_trs(Aop->dims(), Bop->dims(), side_left);
    this->operands.push_back(std::move(Aop));
    this->operands.push_back(std::move(Bop));
  }
  MatrixDims dims() const override {
    return this->operands[1]->dims().repadded(pad);
  }
  size_t output_space_req() const override { return dims().footprint(); }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    blas_check(gpuTtrsm<T>(handle, side_left, lower, trans, unit_diag, mats[0], mats[1], alpha,
                           variant),
               "trsm (MatrixTrsAlloc)");
    return mats[1];
  }
};

// uplo triangle of C = alpha op(A) op(A)^T + beta C into operand C (reference :536-578).
template <typename T>
class MatrixSyrk : public MatrixOp<T> {
 protected:
  bool lower, trans;
  T alpha, beta;
  int variant;

 public:
  MatrixSyrk(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Cop, bool lower,
             bool trans, T alpha, T beta, int variant = RTAT_GEMM_AUTO)
      : MatrixOp<T>({}, 1), lower(lower), trans(trans), alpha(alpha), beta(beta),
        variant(variant) {
    const MatrixDims a = Aop->dims(), c = Cop->dims();
    if (c.m != c.n || (trans ? a.n : a.m) != c.n)
      throw std::invalid_argument("Bad matrix syrk, A is " + std::to_string(a.m) + "x" +
                                  std::to_string(a.n) + ", C is " + std::to_string(c.m) + "x" +
                                  std::to_string(c.n));
    this->operands.push_back(std::move(Aop));
    this->operands.push_back(std::move(Cop));
  }
  MatrixDims dims() const override { return this->operands[1]->dims(); }
  size_t output_space_req() const override { return 0; }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    blas_check(gpuTsyrk<T>(handle, lower, trans, mats[0], mats[1], alpha, beta, variant),
               "syrk (MatrixSyrk)");
    return mats[1];
  }
};

// Fresh, zero-initialised C whose uplo triangle = alpha op(A) op(A)^T (reference :580-617).
template <typename T>
class MatrixSyrkAlloc : public MatrixOp<T> {
 protected:
  bool lower, trans;
  T alpha;
  size_t pad;
  int variant;

 public:
  MatrixSyrkAlloc(std::unique_ptr<MatrixOp<T>> Aop, bool lower, bool trans, T alpha,
                  size_t pad = 1, int variant = RTAT_GEMM_AUTO)
      : MatrixOp<T>({}), lower(lower), trans(trans), alpha(alpha), pad(pad), variant(variant) {
    this->operands.push_back(std::move(Aop));
  }
  MatrixDims dims() const override {
    const MatrixDims a = this->operands[0]->dims();
    const size_t n = trans ? a.n : a.m;
    return MatrixDims(n, n, padded_ld(n, pad));
  }
  size_t output_space_req() const override { return dims().footprint(); }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    this->require_space(out_space, scratch_space, "MatrixSyrkAlloc");
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    Matrix<T> C(out_space, dims());
    blas_check(gpuTgeam<T>(handle, false, false, C, C, C, T(0), T(0)), "geam (zero fill)");
    blas_check(gpuTsyrk<T>(handle, lower, trans, mats[0], C, alpha, T(0), variant),
               "syrk (MatrixSyrkAlloc)");
    return C;
  }
};

// GEMM cut on the host into (mblock, nblock, kblock) sub-products (reference :692-733, never
// instantiated there).  Kept for interface parity; kernel tile-shape variants supersede it.
template <typename T>
class TiledMatrixMult : public MatrixMult<T> {
  int mblock, nblock, kblock;

 public:
  TiledMatrixMult(std::unique_ptr<MatrixOp<T>> Aop, std::unique_ptr<MatrixOp<T>> Bop,
                  std::unique_ptr<MatrixOp<T>> Cop, bool transa, bool transb, T alpha, T beta,
                  int mblock, int nblock, int kblock)
      : MatrixMult<T>(std::move(Aop), std::move(Bop), std::move(Cop), transa, transb, alpha, beta),
        mblock(mblock), nblock(nblock), kblock(kblock) {
    if (mblock <= 0 || nblock <= 0 || kblock <= 0)
      throw std::invalid_argument("TiledMatrixMult: block sizes must be positive");
  }
  Matrix<T> execute(gpu::blasHandle_t handle, Workspace out_space,
                    Workspace scratch_space) override {
    auto mats = this->compute_operands(handle, out_space, scratch_space);
    Matrix<T>&A = mats[0], &B = mats[1], &C = mats[2];
    const int m = (int)C.dims().m, n = (int)C.dims().n;
    const int k = (int)(this->transa ? A.dims().m : A.dims().n);
    for (int i = 0; i < m; i += mblock)
      for (int j = 0; j < n; j += nblock)
        for (int l = 0; l < k; l += kblock) {
          const int ms = std::min(mblock, m - i), ns = std::min(nblock, n - j),
                    ks = std::min(kblock, k - l);
          // op(A)[i.., l..] lives at A[l.., i..] when A is used transposed; same for B.
          Matrix<T> Ab = this->transa ? A.block(l, i, ks, ms) : A.block(i, l, ms, ks);
          Matrix<T> Bb = this->transb ? B.block(j, l, ns, ks) : B.block(l, j, ks, ns);
          Matrix<T> Cb = C.block(i, j, ms, ns);
          blas_check(gpuTgemm<T>(handle, this->transa, this->transb, Ab, Bb, Cb, this->alpha,
                                 l == 0 ? this->beta : T(1)),
                     "gemm (TiledMatrixMult)");
        }
    return C;
  }
};

}  // namespace rtat
