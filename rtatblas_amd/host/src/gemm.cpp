#include "gemm.h"

#include <istream>
#include <ostream>

namespace rtat {

// ---- Tile_Op ---------------------------------------------------------------------------------
Tile_Op::Tile_Op(int id) : id(id) {
  if (rtat_gemm_variant_name(id) == nullptr)
    throw std::runtime_error("Invalid Tile_Op id " + std::to_string(id));
}
Tile_Op::Tile_Op(const std::string& name) {
  for (int v = 0; rtat_gemm_variant_name(v) != nullptr; ++v)
    if (name == rtat_gemm_variant_name(v)) {
      id = v;
      return;
    }
  throw std::runtime_error("Invalid Tile_Op string " + name);
}
Tile_Op::operator std::string() const { return rtat_gemm_variant_name(id); }
std::vector<Tile_Op> Tile_Op::enumerate() {
  std::vector<Tile_Op> all;
  for (int v = 1; rtat_gemm_variant_name(v) != nullptr; ++v) all.push_back(Tile_Op(v));
  return all;
}

// ---- GEMM_Key ----------------------------------------------------------------------------------
GEMM_Key::operator std::string() const {
  return std::string(transa) + "," + std::string(transb) + ",," + std::to_string(m) + "," +
         std::to_string(k) + "," + std::to_string(n);
}
bool GEMM_Key::operator<(const GEMM_Key& rhs) const {
  return std::string(*this) < std::string(rhs);
}
std::ostream& operator<<(std::ostream& os, const GEMM_Key& key) { return os << std::string(key); }

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

std::string read_token(std::istream& is) {
  std::string s;
  is >> s;
  return s;
}

}  // namespace

// ---- GEMM_Options --------------------------------------------------------------------------------
std::vector<GEMM_Options> GEMM_Options::enumerate() {
  std::vector<GEMM_Options> all;
  for (auto a : BLAS_Op::enumerate())
    for (auto b : BLAS_Op::enumerate())
      for (auto c : BLAS_Op::enumerate()) all.emplace_back(a, b, c);
  return all;  // NNN NNT NTN NTT TNN TNT TTN TTT
}
GEMM_Options::operator std::string() const {
  return std::string(transa) + std::string(transb) + std::string(transc);
}
bool GEMM_Options::operator<(const GEMM_Options& o) const {
  return std::string(*this) < std::string(o);
}
std::ostream& operator<<(std::ostream& os, const GEMM_Options opts) {
  return os << std::string(opts);
}
std::istream& operator>>(std::istream& is, GEMM_Options& opts) {
  const std::string s = read_token(is);
  if (s.size() != 3) {
    is.setstate(std::ios::failbit);
    return is;
  }
  opts = GEMM_Options(BLAS_Op(s[0]), BLAS_Op(s[1]), BLAS_Op(s[2]));
  return is;
}
template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, false, false, false, RTAT_GEMM_AUTO);
}

// ---- GEMM_Options_Pad ------------------------------------------------------------------------------
std::vector<GEMM_Options_Pad> GEMM_Options_Pad::enumerate() {
  std::vector<GEMM_Options_Pad> all;
  for (auto a : BLAS_Op::enumerate())
    for (auto b : BLAS_Op::enumerate())
      for (auto c : BLAS_Op::enumerate())
        for (auto pa : Pad_Op::enumerate())
          for (auto pb : Pad_Op::enumerate())
            for (auto pc : Pad_Op::enumerate()) all.emplace_back(a, pa, b, pb, c, pc);
  return all;
}
GEMM_Options_Pad::operator std::string() const {
  return std::string(transa) + std::string(transb) + std::string(transc) + std::string(pada) +
         std::string(padb) + std::string(padc);
}
bool GEMM_Options_Pad::operator<(const GEMM_Options_Pad& o) const {
  return std::string(*this) < std::string(o);
}
std::ostream& operator<<(std::ostream& os, const GEMM_Options_Pad opts) {
  return os << std::string(opts);
}
std::istream& operator>>(std::istream& is, GEMM_Options_Pad& opts) {
  const std::string s = read_token(is);
  if (s.size() != 6) {
    is.setstate(std::ios::failbit);
    return is;
  }
  opts = GEMM_Options_Pad(BLAS_Op(s[0]), Pad_Op(s[3]), BLAS_Op(s[1]), Pad_Op(s[4]), BLAS_Op(s[2]),
                          Pad_Op(s[5]));
  return is;
}
template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options_Pad::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, pada == Pad_Op::PAD, padb == Pad_Op::PAD,
                            padc == Pad_Op::PAD, RTAT_GEMM_AUTO);
}

// ---- GEMM_Options_Tile -----------------------------------------------------------------------------
std::vector<GEMM_Options_Tile> GEMM_Options_Tile::enumerate() {
  std::vector<GEMM_Options_Tile> all;
  for (auto a : BLAS_Op::enumerate())
    for (auto b : BLAS_Op::enumerate())
      for (auto c : BLAS_Op::enumerate())
        for (auto t : Tile_Op::enumerate()) all.emplace_back(a, b, c, t);
  return all;
}
GEMM_Options_Tile::operator std::string() const {
  return std::string(transa) + std::string(transb) + std::string(transc) + "/" + std::string(tile);
}
bool GEMM_Options_Tile::operator<(const GEMM_Options_Tile& o) const {
  return std::string(*this) < std::string(o);
}
std::ostream& operator<<(std::ostream& os, const GEMM_Options_Tile opts) {
  return os << std::string(opts);
}
std::istream& operator>>(std::istream& is, GEMM_Options_Tile& opts) {
  const std::string s = read_token(is);
  if (s.size() < 5 || s[3] != '/') {
    is.setstate(std::ios::failbit);
    return is;
  }
  opts = GEMM_Options_Tile(BLAS_Op(s[0]), BLAS_Op(s[1]), BLAS_Op(s[2]), Tile_Op(s.substr(4)));
  return is;
}
template <typename T>
std::unique_ptr<MatrixOp<T>> GEMM_Options_Tile::form_operation(GEMM_Inputs<T> params) {
  return build_gemm_tree<T>(params, transa == BLAS_Op::TRANS, transb == BLAS_Op::TRANS,
                            transc == BLAS_Op::TRANS, false, false, false, tile.id);
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
template std::unique_ptr<MatrixOp<double>> GEMM_Options_Tile::form_operation(GEMM_Inputs<double>);
template std::unique_ptr<MatrixOp<float>> GEMM_Options_Tile::form_operation(GEMM_Inputs<float>);

}  // namespace rtat
