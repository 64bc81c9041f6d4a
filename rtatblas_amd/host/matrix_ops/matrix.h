// Column-major matrix views over a Workspace (reference src/matrix_ops/matrix.h).
#pragma once
#include <ostream>
#include <stdexcept>

#include "workspace.h"

namespace rtat {

struct MatrixDims {
  size_t m = 0, n = 0, ld = 0;
  MatrixDims() = default;
  MatrixDims(size_t m, size_t n, size_t ld) : m(m), n(n), ld(ld) {
    if (ld < m) throw std::invalid_argument("ld < m in MatrixDims");
  }
  // Elements the matrix spans in memory.
  size_t footprint() const { return ld * n; }
  friend std::ostream& operator<<(std::ostream& os, const MatrixDims& d) {
    return os << "(" << d.m << "," << d.n << "," << d.ld << ")";
  }
};

// Leading dimension of an m-row result padded to a multiple of `pad` elements.
inline size_t padded_ld(size_t m, size_t pad) { return (m + pad - 1) / pad * pad; }

template <typename T>
class Matrix {
 public:
  Matrix() = default;
  Matrix(Workspace home, MatrixDims dims) : home(home), dimensions(dims) {}
  Matrix(Workspace home, size_t m, size_t n, size_t ld) : Matrix(home, MatrixDims(m, n, ld)) {}

  // nrows x ncols window starting at (row, col), same leading dimension.  (The reference,
  // matrix.h:40-48, hands an element offset to a constructor that expects bytes; this one
  // converts.)
  Matrix block(size_t row, size_t col, size_t nrows, size_t ncols) {
    if (row + nrows > dimensions.m || col + ncols > dimensions.n)
      throw std::out_of_range("Matrix::block outside the matrix");
    MatrixDims d(nrows, ncols, dimensions.ld);
    const size_t first = row + col * dimensions.ld;
    const size_t span = ncols == 0 ? 0 : (ncols - 1) * dimensions.ld + nrows;
    Workspace w(home, first * sizeof(T), span * sizeof(T));
    return Matrix(w, d);
  }

  size_t footprint() const { return dimensions.footprint(); }
  const MatrixDims dims() const { return dimensions; }
  T* ptr() const { return (T*)home; }

 private:
  Workspace home;
  MatrixDims dimensions;
};

}  // namespace rtat
