// Blocked fp64 triangular solve for gfx950.
//
// Serves gpuTtrsm of the reference (src/matrix_ops/matrixop.h:78-109), which forwards to
// hipblasDtrsm: solve op(A) X = alpha B (left) or X op(A) = alpha B (right) in place in B.
//
// Method
//   1. The NB x NB diagonal blocks of A (NB = 128) are inverted, one workgroup per block,
//      entirely in LDS (unblocked in-place triangular inversion), into scratch.
//   2. The solve recurses on halves of the triangular dimension: solve one half, update the
//      other with one large-k DGEMM (alpha = -1, beta = 1) on the MFMA core, solve the other
//      half.  A leaf (<= NB) is X_i = op(inv(A_ii)) B_i, also on the MFMA core, in place:
//      the leaf uses a single tile row (left) / tile column (right), so every workgroup
//      reads exactly the part of B it later overwrites, and reads it before writing.
//   All sixteen side / uplo / trans / diag combinations run natively: trans flips the
//   effective triangle and is passed to the DGEMM as an operand flag; inv(op(T)) = op(inv(T)).
//
// Flop count used for reporting: m*m*n (left), m*n*n (right).
#include "common.h"

namespace rtat_native {

constexpr int NB = 128;

typedef double d2_t __attribute__((ext_vector_type(2)));

constexpr int TRTRI_LD = NB + 1;  // odd stride: a row and a column walk are both conflict free
constexpr size_t TRTRI_LDS_BYTES = (size_t)(NB * TRTRI_LD + 3 * NB) * sizeof(double);

// One workgroup inverts one diagonal block; lane i owns row i.  The block is held in LDS as
// a LOWER triangular matrix (an upper block is transposed on the way in and out), inverted
// in place column by column from the last to the first, and written out as a full NB x NB
// square whose other triangle is zero, so it can feed a plain DGEMM.
//
// Column j of the inverse below the diagonal is -inv(L22) * L(j+1:, j) / L(j,j), where
// inv(L22) already sits in L(j+1:, j+1:).  Lane i only ever reads and writes its own row of
// L; the one thing that crosses lanes is the column vector L(:, j), handed over through a
// double-buffered copy, so one barrier per column is enough.  The dot product of row i runs
// over k = j+1 .. i; it is padded to the same 4-aligned range for the whole wavefront, the
// padding multiplying zeros (entries above the diagonal of L, entries up to j of the
// column copy), so the loop is branch free and four independent sums hide the LDS latency.
__global__ __launch_bounds__(NB) void trtri_kernel(const double* A, long lda, int na, int lower,
                                                  int unit, double* out) {
  extern __shared__ __align__(16) double sm[];
  constexpr int LD = TRTRI_LD;
  double* L = sm;                 // NB x NB, column-major, ld = LD
  double* col = sm + NB * LD;     // 2 x NB: original column j, zero up to row j
  double* dinv = col + 2 * NB;    // reciprocals of the diagonal
  const int blk = blockIdx.x;
  const int b0 = blk * NB;
  const int nb = (na - b0 < NB) ? na - b0 : NB;
  const int i = threadIdx.x;
  const double* Ab = A + b0 + (long)b0 * lda;

  // Load the strict triangle (coalesced along the stored columns), zero the rest; rows and
  // columns past the end of A become identity.
  for (int c = 0; c < NB; ++c) {
    const bool inside = i < nb && c < nb;
    double v = 0.0;
    if (lower) {
      if (inside && c < i) v = Ab[i + (long)c * lda];
      L[i + c * LD] = v;
    } else {
      if (inside && i < c) v = Ab[i + (long)c * lda];
      L[c + i * LD] = v;
    }
  }
  {
    double d = 1.0;
    if (i < nb && !unit) d = Ab[i + (long)i * lda];
    d = 1.0 / d;
    dinv[i] = d;
    L[i + i * LD] = d;  // written by the lane that zeroed it above
  }
  __syncthreads();

  const int wave_end = (i | 63) + 1;  // one past the last row of this wavefront
  for (int j = NB - 1; j >= 0; --j) {
    double* cj = col + (j & 1) * NB;
    cj[i] = i > j ? L[i + j * LD] : 0.0;
    __syncthreads();
    if (wave_end - 1 > j) {
      double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
      const double* Li = L + i;
      for (int k = (j + 1) & ~3; k < wave_end; k += 4) {
        const d2_t c01 = *reinterpret_cast<const d2_t*>(cj + k);
        const d2_t c23 = *reinterpret_cast<const d2_t*>(cj + k + 2);
        s0 += Li[(k + 0) * LD] * c01[0];
        s1 += Li[(k + 1) * LD] * c01[1];
        s2 += Li[(k + 2) * LD] * c23[0];
        s3 += Li[(k + 3) * LD] * c23[1];
      }
      if (i > j) L[i + j * LD] = -((s0 + s1) + (s2 + s3)) * dinv[j];
    }
  }
  __syncthreads();

  double* O = out + (long)blk * NB * NB;
  for (int k = 0; k < NB; ++k) {
    // lower: O(i,k) = L(i,k); upper: O(i,k) = L(k,i).
    O[i + k * NB] = lower ? L[i + k * LD] : L[k + i * LD];
  }
}

struct TrsmCtx {
  rtat_native_handle* h;
  bool left, lower, trans;
  int m, n;
  const double* A;
  int lda;
  double* B;
  int ldb;
  const double* inv;
  int variant;
  rtat_status_t st;
};

static inline int split_point(int lo, int hi) {
  const int blocks = (hi - lo + NB - 1) / NB;
  return lo + NB * ((blocks + 1) / 2);
}

// Block op(A)[I, J] as a DGEMM operand: pointer into A plus the transpose flag.
static inline const double* a_block(const TrsmCtx& c, int i0, int j0) {
  return c.trans ? c.A + j0 + (long)i0 * c.lda : c.A + i0 + (long)j0 * c.lda;
}

static void solve_range(TrsmCtx& c, int lo, int hi) {
  if (c.st != RTAT_STATUS_SUCCESS || hi <= lo) return;
  const int len = hi - lo;
  if (len <= NB) {
    const double* invb = c.inv + (long)(lo / NB) * NB * NB;
    if (c.left) {
      double* Bi = c.B + lo;
      const long cus = c.h->compute_units > 0 ? c.h->compute_units : 256;
      const int v = ((long)((c.n + 127) / 128) >= cus) ? RTAT_GEMM_T128x128 : RTAT_GEMM_T128x64;
      c.st = launch_dgemm(c.h, c.trans, false, len, c.n, len, 1.0, invb, NB, Bi, c.ldb, 0.0, Bi,
                          c.ldb, 0, v);
    } else {
      double* Bj = c.B + (long)lo * c.ldb;
      c.st = launch_dgemm(c.h, false, c.trans, c.m, len, len, 1.0, Bj, c.ldb, invb, NB, 0.0, Bj,
                          c.ldb, 0, RTAT_GEMM_T128x128);
    }
    return;
  }
  const int mid = split_point(lo, hi);
  const bool eff_lower = c.lower != c.trans;
  if (c.left) {
    if (eff_lower) {
      solve_range(c, lo, mid);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_dgemm(c.h, c.trans, false, hi - mid, c.n, mid - lo, -1.0,
                            a_block(c, mid, lo), c.lda, c.B + lo, c.ldb, 1.0, c.B + mid, c.ldb,
                            0, c.variant);
      solve_range(c, mid, hi);
    } else {
      solve_range(c, mid, hi);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_dgemm(c.h, c.trans, false, mid - lo, c.n, hi - mid, -1.0,
                            a_block(c, lo, mid), c.lda, c.B + mid, c.ldb, 1.0, c.B + lo, c.ldb,
                            0, c.variant);
      solve_range(c, lo, mid);
    }
  } else {
    double* Blo = c.B + (long)lo * c.ldb;
    double* Bmid = c.B + (long)mid * c.ldb;
    if (eff_lower) {
      solve_range(c, mid, hi);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_dgemm(c.h, false, c.trans, c.m, mid - lo, hi - mid, -1.0, Bmid, c.ldb,
                            a_block(c, mid, lo), c.lda, 1.0, Blo, c.ldb, 0, c.variant);
      solve_range(c, lo, mid);
    } else {
      solve_range(c, lo, mid);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_dgemm(c.h, false, c.trans, c.m, hi - mid, mid - lo, -1.0, Blo, c.ldb,
                            a_block(c, lo, mid), c.lda, 1.0, Bmid, c.ldb, 0, c.variant);
      solve_range(c, mid, hi);
    }
  }
}

size_t trsm_workspace_bytes(int na) {
  if (na <= 0) return 0;
  return (size_t)((na + NB - 1) / NB) * NB * NB * sizeof(double);
}

rtat_status_t launch_dtrsm(rtat_native_handle* h, bool left, bool lower, bool trans, bool unit,
                           int m, int n, double alpha, const double* A, int lda, double* B,
                           int ldb, int variant) {
  if (m < 0 || n < 0 || ldb < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (variant < 0 || variant >= RTAT_GEMM_VARIANT_COUNT) return RTAT_STATUS_INVALID_VALUE;
  const int na = left ? m : n;
  if (lda < (na > 1 ? na : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (B == nullptr) return RTAT_STATUS_INVALID_VALUE;
  if (alpha == 0.0)
    return launch_geam<double>(h, false, false, m, n, 0.0, nullptr, 0, 0.0, nullptr, 0, B, ldb);
  if (A == nullptr) return RTAT_STATUS_INVALID_VALUE;

  const size_t need = trsm_workspace_bytes(na);
  double* inv = static_cast<double*>(acquire_workspace(h, need));
  if (inv == nullptr) return RTAT_STATUS_ALLOC_FAILED;

  static bool configured = false;
  const size_t lds_bytes = TRTRI_LDS_BYTES;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(trtri_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess) {
      (void)hipGetLastError();
      return RTAT_STATUS_NOT_SUPPORTED;
    }
    configured = true;
  }
  const int nblk = (na + NB - 1) / NB;
  hipLaunchKernelGGL(trtri_kernel, dim3(nblk), dim3(NB), lds_bytes, h->stream, A, (long)lda, na,
                     lower ? 1 : 0, unit ? 1 : 0, inv);
  rtat_status_t st = launch_status();
  if (st != RTAT_STATUS_SUCCESS) return st;

  if (alpha != 1.0) {
    st = launch_geam<double>(h, false, false, m, n, alpha, B, ldb, 0.0, nullptr, 0, B, ldb);
    if (st != RTAT_STATUS_SUCCESS) return st;
  }
  TrsmCtx c{h, left, lower, trans, m, n, A, lda, B, ldb, inv, variant, RTAT_STATUS_SUCCESS};
  solve_range(c, 0, na);
  return c.st;
}

}  // namespace rtat_native
