// Column-major matrix views over a Workspace (reference src/matrix_ops/matrix.h).
#pragma once
#include <ostream>
#include <stdexcept>

#include "workspace.h"

namespace rtat {

// Leading dimension of an m-row result padded to a multiple of `pad` elements.
inline size_t padded_ld(size_t m, size_t pad) { return (m + pad - 1) / pad * pad; }

// Shape of a column-major matrix: m rows, n columns, ld elements between columns.
struct MatrixDims {
  size_t m = 0, n = 0, ld = 0;

  MatrixDims() = default;
  MatrixDims(size_t m, size_t n, size_t ld) : m(m), n(n), ld(ld) {
    if (ld < m) throw std::invalid_argument("ld < m in MatrixDims");
  }

  // Elements the matrix spans in memory, padding rows included (what scratch must hold).
  size_t footprint() const { return ld * n; }
  // Elements from the first to one past the last one that is ever touched.
  size_t span() const { return n == 0 ? 0 : (n - 1) * ld + m; }
  // Shape of the transpose, tightly packed or with its leading dimension padded.
  MatrixDims transposed(size_t pad = 1) const { return MatrixDims(n, m, padded_ld(n, pad)); }
  // Same logical shape with the leading dimension padded.
  MatrixDims repadded(size_t pad) const { return MatrixDims(m, n, padded_ld(m, pad)); }

  bool operator==(const MatrixDims& o) const { return m == o.m && n == o.n && ld == o.ld; }
  bool operator!=(const MatrixDims& o) const { return !(*this == o); }
  friend std::ostream& operator<<(std::ostream& os, const MatrixDims& d) {
    return os << "(" << d.m << "," << d.n << "," << d.ld << ")";
  }
};

template <typename T>
class Matrix {
  Workspace home;
  MatrixDims shape;

 public:
  Matrix() = default;
  Matrix(Workspace home, MatrixDims dims) : home(home), shape(dims) {}
  Matrix(Workspace home, size_t m, size_t n, size_t ld) : Matrix(home, MatrixDims(m, n, ld)) {}

  const MatrixDims dims() const { return shape; }
  size_t footprint() const { return shape.footprint(); }
  T* ptr() const { return (T*)home; }
  // Address of element (row, col).
  T* at(size_t row, size_t col) const { return ptr() + row + col * shape.ld; }

  // The nrows x ncols window whose top-left element is (row, col); it shares this matrix's
  // memory and leading dimension.  (The reference's block, matrix.h:40-48, hands an element
  // offset to a constructor that expects bytes; this one converts.)
  Matrix block(size_t row, size_t col, size_t nrows, size_t ncols) {
    if (row + nrows > shape.m || col + ncols > shape.n)
      throw std::out_of_range("Matrix::block outside the matrix");
    const MatrixDims window(nrows, ncols, shape.ld);
    return Matrix(Workspace(home, (row + col * shape.ld) * sizeof(T), window.span() * sizeof(T)),
                  window);
  }
};

}  // namespace rtat
