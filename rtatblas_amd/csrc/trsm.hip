// Blocked triangular solve for gfx950 (double and float from one template).
//
// Serves gpuTtrsm of the reference (src/matrix_ops/matrixop.h:78-109), which forwards to
// hipblas{D,S}trsm: solve op(A) X = alpha B (left) or X op(A) = alpha B (right) in place in B.
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

constexpr int TRTRI_LD = NB + 1;  // odd stride: a row walk and a column walk are both conflict free
constexpr int TRTRI_THREADS = 256;
constexpr int TRTRI_SB = 16;      // diagonal sub-blocks inverted by substitution
constexpr size_t TRTRI_LDS_ELEMS = (size_t)(NB * TRTRI_LD + 3 * NB);

// One level of the blocked inversion of a lower triangular L held in LDS: every 2B x 2B
// diagonal block [L11 0; L21 L22] whose B x B diagonal blocks already hold their inverses
// gets its off-diagonal block replaced by -inv(L22) L21 inv(L11).  All 256 lanes work: each
// owns a TR x TC register tile of one block pair; the intermediate L21 inv(L11) is parked
// in the upper right 64 x 64 quadrant of L, which a lower triangular matrix never uses.
template <class T, int B, int TR, int TC>
__device__ inline void trtri_level(T* L, int t) {
  constexpr int LD = TRTRI_LD;
  constexpr int TILES_R = B / TR, TILES_PER_PAIR = TILES_R * (B / TC);
  static_assert(TILES_PER_PAIR * (NB / (2 * B)) == TRTRI_THREADS, "one register tile per lane");
  const int pair = t / TILES_PER_PAIR, q = t % TILES_PER_PAIR;
  // Lane rows are r0, r0 + TILES_R, ...: neighbouring lanes read neighbouring LDS words.
  const int r0 = q % TILES_R, c0 = TC * (q / TILES_R);
  const int o = 2 * B * pair;
  T acc[TR][TC];

  // W = L21 * inv(L11); inv(L11)(k, c) is zero for k < c.
  const T* l21 = L + (o + B + r0) + o * LD;  // (r, k) at l21[r + k * LD]
  const T* i11 = L + o + (o + c0) * LD;      // (k, c) at i11[k + c * LD]
#pragma unroll
  for (int r = 0; r < TR; ++r)
#pragma unroll
    for (int c = 0; c < TC; ++c) acc[r][c] = T(0);
#pragma unroll 4
  for (int k = c0; k < B; ++k) {
    T a[TR], bb[TC];
#pragma unroll
    for (int r = 0; r < TR; ++r) a[r] = l21[r * TILES_R + k * LD];
#pragma unroll
    for (int c = 0; c < TC; ++c) bb[c] = i11[k + c * LD];
#pragma unroll
    for (int r = 0; r < TR; ++r)
#pragma unroll
      for (int c = 0; c < TC; ++c) acc[r][c] += a[r] * bb[c];
  }
  T* W = L + B * pair + (NB / 2) * LD;  // W(r, c) of this pair at W[r + c * LD]
#pragma unroll
  for (int r = 0; r < TR; ++r)
#pragma unroll
    for (int c = 0; c < TC; ++c) W[(r0 + r * TILES_R) + (c0 + c) * LD] = acc[r][c];
  __syncthreads();

  // X = -inv(L22) * W, into the place of L21 (nobody reads L21 any more).
  const T* i22 = L + (o + B + r0) + (o + B) * LD;  // (r, k) at i22[r + k * LD]
  const T* Wc = W + c0 * LD;                       // (k, c) at Wc[k + c * LD]
#pragma unroll
  for (int r = 0; r < TR; ++r)
#pragma unroll
    for (int c = 0; c < TC; ++c) acc[r][c] = T(0);
#pragma unroll 4
  for (int k = 0; k < B; ++k) {
    T a[TR], bb[TC];
#pragma unroll
    for (int r = 0; r < TR; ++r) a[r] = i22[r * TILES_R + k * LD];
#pragma unroll
    for (int c = 0; c < TC; ++c) bb[c] = Wc[k + c * LD];
#pragma unroll
    for (int r = 0; r < TR; ++r)
#pragma unroll
      for (int c = 0; c < TC; ++c) acc[r][c] += a[r] * bb[c];
  }
  T* x = L + (o + B + r0) + (o + c0) * LD;
#pragma unroll
  for (int r = 0; r < TR; ++r)
#pragma unroll
    for (int c = 0; c < TC; ++c) x[r * TILES_R + c * LD] = -acc[r][c];
  __syncthreads();
}

// One workgroup inverts one NB x NB diagonal block.  The block is held in LDS as a LOWER
// triangular matrix (an upper block is transposed on the way in and out) and written out as
// a full NB x NB square whose other triangle is zero, so it can feed a plain DGEMM.
//   1. The eight 16 x 16 diagonal sub-blocks are inverted by column substitution, all in
//      lockstep: column j of an inverse below the diagonal is -inv(L22) L(j+1:, j) / L(j,j),
//      where inv(L22) already sits in L(j+1:, j+1:).  Lane i only reads and writes its own
//      row; the column L(:, j) crosses lanes through a double-buffered copy (one barrier per
//      column), zero up to row j so that the 16-term dot product needs no bounds.
//   2. Three doubling levels (16 -> 32 -> 64 -> 128) fill in the off-diagonal blocks with
//      small register-tiled matrix products (trtri_level).
template <class T>
__global__ __launch_bounds__(TRTRI_THREADS) void trtri_kernel(const T* A, long lda, int na, int lower,
                                                             int unit, T* out) {
  extern __shared__ __align__(16) unsigned char sm_raw[];
  T* sm = reinterpret_cast<T*>(sm_raw);
  constexpr int LD = TRTRI_LD, SB = TRTRI_SB;
  T* L = sm;                 // NB x NB, column-major, ld = LD
  T* col = sm + NB * LD;     // 2 x NB column hand-over
  T* dinv = col + 2 * NB;    // reciprocals of the diagonal
  const int blk = blockIdx.x;
  const int b0 = blk * NB;
  const int nb = (na - b0 < NB) ? na - b0 : NB;
  const int t = threadIdx.x;
  const int i = t & (NB - 1), half = t >> 7;  // two lanes per row
  const T* Ab = A + b0 + (long)b0 * lda;

  // Load the strict triangle (coalesced along the stored columns), zero the rest; rows and
  // columns past the end of A become identity.  Eight columns are in flight per lane.
  for (int c8 = half; c8 < NB; c8 += 16) {
    T v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c8 + 2 * u;
      const bool wanted = i < nb && c < nb && (lower ? c < i : i < c);
      v[u] = wanted ? Ab[i + (long)c * lda] : T(0);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c8 + 2 * u;
      if (lower) L[i + c * LD] = v[u];
      else L[c + i * LD] = v[u];
    }
  }
  __syncthreads();
  if (half == 0) {
    T d = T(1);
    if (i < nb && !unit) d = Ab[i + (long)i * lda];
    d = T(1) / d;
    dinv[i] = d;
    L[i + i * LD] = d;
  }
  __syncthreads();

  const int bi = i & (SB - 1), s0 = i & ~(SB - 1);  // row within its sub-block, sub-block start
  for (int j = SB - 1; j >= 0; --j) {
    T* cj = col + (j & 1) * NB;
    if (half == 0) cj[i] = bi > j ? L[i + (s0 + j) * LD] : T(0);
    __syncthreads();
    if (half == 0 && bi > j) {
      T e0 = T(0), e1 = T(0);
#pragma unroll
      for (int k = 0; k < SB; k += 2) {
        e0 += L[i + (s0 + k) * LD] * cj[s0 + k];
        e1 += L[i + (s0 + k + 1) * LD] * cj[s0 + k + 1];
      }
      L[i + (s0 + j) * LD] = -(e0 + e1) * dinv[s0 + j];
    }
  }
  __syncthreads();

  trtri_level<T, 16, 2, 2>(L, t);
  trtri_level<T, 32, 4, 2>(L, t);
  trtri_level<T, 64, 4, 4>(L, t);

  T* O = out + (long)blk * NB * NB;
  for (int k = half; k < NB; k += 2) {
    // lower: O(i,k) = L(i,k) for k <= i; upper: O(i,k) = L(k,i) for i <= k; zero elsewhere.
    T v = T(0);
    if (lower) {
      if (k <= i) v = L[i + k * LD];
    } else {
      if (i <= k) v = L[k + i * LD];
    }
    O[i + k * NB] = v;
  }
}

template <class T>
struct TrsmCtx {
  rtat_native_handle* h;
  bool left, lower, trans;
  int m, n;
  const T* A;
  int lda;
  T* B;
  int ldb;
  const T* inv;
  int variant;
  rtat_status_t st;
};

static inline int split_point(int lo, int hi) {
  const int blocks = (hi - lo + NB - 1) / NB;
  return lo + NB * ((blocks + 1) / 2);
}

// Block op(A)[I, J] as a GEMM operand: pointer into A plus the transpose flag.
template <class T>
static inline const T* a_block(const TrsmCtx<T>& c, int i0, int j0) {
  return c.trans ? c.A + j0 + (long)i0 * c.lda : c.A + i0 + (long)j0 * c.lda;
}

template <class T>
static void solve_range(TrsmCtx<T>& c, int lo, int hi) {
  if (c.st != RTAT_STATUS_SUCCESS || hi <= lo) return;
  const int len = hi - lo;
  if (len <= NB) {
    const T* invb = c.inv + (long)(lo / NB) * NB * NB;
    if (c.left) {
      T* Bi = c.B + lo;
      const long cus = c.h->compute_units > 0 ? c.h->compute_units : 256;
      const int v = ((long)((c.n + 127) / 128) >= cus) ? RTAT_GEMM_T128x128 : RTAT_GEMM_T128x64;
      c.st = launch_gemm<T>(c.h, c.trans, false, len, c.n, len, T(1), invb, NB, Bi, c.ldb, T(0), Bi,
                          c.ldb, 0, v);
    } else {
      T* Bj = c.B + (long)lo * c.ldb;
      c.st = launch_gemm<T>(c.h, false, c.trans, c.m, len, len, T(1), Bj, c.ldb, invb, NB, T(0), Bj,
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
        c.st = launch_gemm<T>(c.h, c.trans, false, hi - mid, c.n, mid - lo, T(-1),
                            a_block(c, mid, lo), c.lda, c.B + lo, c.ldb, T(1), c.B + mid, c.ldb,
                            0, c.variant);
      solve_range(c, mid, hi);
    } else {
      solve_range(c, mid, hi);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_gemm<T>(c.h, c.trans, false, mid - lo, c.n, hi - mid, T(-1),
                            a_block(c, lo, mid), c.lda, c.B + mid, c.ldb, T(1), c.B + lo, c.ldb,
                            0, c.variant);
      solve_range(c, lo, mid);
    }
  } else {
    T* Blo = c.B + (long)lo * c.ldb;
    T* Bmid = c.B + (long)mid * c.ldb;
    if (eff_lower) {
      solve_range(c, mid, hi);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_gemm<T>(c.h, false, c.trans, c.m, mid - lo, hi - mid, T(-1), Bmid, c.ldb,
                            a_block(c, mid, lo), c.lda, T(1), Blo, c.ldb, 0, c.variant);
      solve_range(c, lo, mid);
    } else {
      solve_range(c, lo, mid);
      if (c.st == RTAT_STATUS_SUCCESS)
        c.st = launch_gemm<T>(c.h, false, c.trans, c.m, hi - mid, mid - lo, T(-1), Blo, c.ldb,
                            a_block(c, lo, mid), c.lda, T(1), Bmid, c.ldb, 0, c.variant);
      solve_range(c, mid, hi);
    }
  }
}

size_t trsm_workspace_bytes(int na) {
  if (na <= 0) return 0;
  return (size_t)((na + NB - 1) / NB) * NB * NB * sizeof(double);  // float needs half of it
}

template <class T>
rtat_status_t launch_trsm(rtat_native_handle* h, bool left, bool lower, bool trans, bool unit,
                          int m, int n, T alpha, const T* A, int lda, T* B, int ldb,
                          int variant) {
  if (m < 0 || n < 0 || ldb < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (variant < 0 || variant >= RTAT_GEMM_VARIANT_COUNT) return RTAT_STATUS_INVALID_VALUE;
  const int na = left ? m : n;
  if (lda < (na > 1 ? na : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (B == nullptr) return RTAT_STATUS_INVALID_VALUE;
  if (alpha == T(0))
    return launch_geam<T>(h, false, false, m, n, T(0), nullptr, 0, T(0), nullptr, 0, B, ldb);
  if (A == nullptr) return RTAT_STATUS_INVALID_VALUE;

  const size_t need = (size_t)((na + NB - 1) / NB) * NB * NB * sizeof(T);
  T* inv = static_cast<T*>(acquire_workspace(h, need));
  if (inv == nullptr) return RTAT_STATUS_ALLOC_FAILED;

  static bool configured = false;
  const size_t lds_bytes = TRTRI_LDS_ELEMS * sizeof(T);
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(trtri_kernel<T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess) {
      (void)hipGetLastError();
      return RTAT_STATUS_NOT_SUPPORTED;
    }
    configured = true;
  }
  const int nblk = (na + NB - 1) / NB;
  hipLaunchKernelGGL(trtri_kernel<T>, dim3(nblk), dim3(TRTRI_THREADS), lds_bytes, h->stream, A,
                     (long)lda, na, lower ? 1 : 0, unit ? 1 : 0, inv);
  rtat_status_t st = launch_status();
  if (st != RTAT_STATUS_SUCCESS) return st;

  if (alpha != T(1)) {
    st = launch_geam<T>(h, false, false, m, n, alpha, B, ldb, T(0), nullptr, 0, B, ldb);
    if (st != RTAT_STATUS_SUCCESS) return st;
  }
  TrsmCtx<T> c{h, left, lower, trans, m, n, A, lda, B, ldb, inv, variant, RTAT_STATUS_SUCCESS};
  solve_range(c, 0, na);
  return c.st;
}

template rtat_status_t launch_trsm<double>(rtat_native_handle*, bool, bool, bool, bool, int, int,
                                           double, const double*, int, double*, int, int);
template rtat_status_t launch_trsm<float>(rtat_native_handle*, bool, bool, bool, bool, int, int,
                                          float, const float*, int, float*, int, int);

}  // namespace rtat_native
