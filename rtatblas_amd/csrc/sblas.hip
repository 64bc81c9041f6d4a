// Single-precision GEMM / SYRK / TRSM: plain LDS-tiled VALU kernels so that the float
// instantiations of the reference's templates (gpuTgemm<float> ... in
// src/matrix_ops/matrixop.h:33-43, 64-73, 96-105) have something to call.  Correct for every
// argument combination, not tuned: the tuned path of this library is fp64.
#include "common.h"

namespace rtat_native {

constexpr int ST = 64;   // C tile edge
constexpr int SK = 16;   // k step

// 256 lanes, each owns a 4 x 4 patch of the 64 x 64 tile.
__global__ __launch_bounds__(256) void sgemm_kernel(int ta, int tb, int m, int n, int k,
                                                   float alpha, const float* A, long lda,
                                                   const float* B, long ldb, float beta,
                                                   float* C, long ldc, int tri) {
  __shared__ float sa[SK][ST + 1];
  __shared__ float sb[SK][ST + 1];
  const int m0 = blockIdx.x * ST, n0 = blockIdx.y * ST;
  if (tri == 1 && m0 + ST - 1 < n0) return;
  if (tri == 2 && m0 > n0 + ST - 1) return;
  const int t = threadIdx.x, ti = t % 16, tj = t / 16;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += SK) {
    for (int e = t; e < ST * SK; e += 256) {
      const int r = e % ST, kk = e / ST;
      const int gi = m0 + r, gj = n0 + r, gk = k0 + kk;
      float va = 0.f, vb = 0.f;
      if (gk < k) {
        if (gi < m) va = ta ? A[gk + (long)gi * lda] : A[gi + (long)gk * lda];
        if (gj < n) vb = tb ? B[gj + (long)gk * ldb] : B[gk + (long)gj * ldb];
      }
      sa[kk][r] = va;
      sb[kk][r] = vb;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < SK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) { a[x] = sa[kk][ti + 16 * x]; b[x] = sb[kk][tj + 16 * x]; }
#pragma unroll
      for (int y = 0; y < 4; ++y)
#pragma unroll
        for (int x = 0; x < 4; ++x) acc[y][x] = fmaf(a[x], b[y], acc[y][x]);
    }
    __syncthreads();
  }
  for (int y = 0; y < 4; ++y) {
    const int col = n0 + tj + 16 * y;
    if (col >= n) continue;
    for (int x = 0; x < 4; ++x) {
      const int row = m0 + ti + 16 * x;
      if (row >= m) continue;
      if (tri == 1 && row < col) continue;
      if (tri == 2 && row > col) continue;
      float* c = C + row + (long)col * ldc;
      float v = alpha * acc[y][x];
      if (beta != 0.f) v += beta * *c;
      *c = v;
    }
  }
}

// One lane per right-hand side (a column of B on the left side, a row on the right) doing
// plain substitution; all lanes walk A in the same order so its reads are broadcasts.
__global__ __launch_bounds__(256) void strsm_kernel(int left, int lower, int trans, int unit,
                                                   int m, int n, float alpha, const float* A,
                                                   long lda, float* B, long ldb) {
  const int rhs = blockIdx.x * 256 + threadIdx.x;
  const int nrhs = left ? n : m, na = left ? m : n;
  if (rhs >= nrhs) return;
  auto a = [&](int i, int j) { return trans ? A[j + (long)i * lda] : A[i + (long)j * lda]; };
  auto b = [&](int q) -> float& {  // q-th unknown of this right-hand side
    return left ? B[q + (long)rhs * ldb] : B[rhs + (long)q * ldb];
  };
  const bool eff_lower = (lower != 0) != (trans != 0);
  // left:  sum_k opA(q,k) x_k = b_q ; right: sum_k x_k opA(k,q) = b_q.
  // Forward order when the coupling matrix seen by x is lower (left) / upper (right).
  const bool forward = left ? eff_lower : !eff_lower;
  for (int s = 0; s < na; ++s) {
    const int q = forward ? s : na - 1 - s;
    float v = alpha * b(q);
    for (int u = 0; u < s; ++u) {
      const int kk = forward ? u : na - 1 - u;
      v -= (left ? a(q, kk) : a(kk, q)) * b(kk);
    }
    if (!unit) v /= a(q, q);
    b(q) = v;
  }
}

rtat_status_t launch_sgemm(rtat_native_handle* h, bool ta, bool tb, int m, int n, int k,
                           float alpha, const float* A, int lda, const float* B, int ldb,
                           float beta, float* C, int ldc, int tri) {
  if (m < 0 || n < 0 || k < 0 || ldc < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (C == nullptr) return RTAT_STATUS_INVALID_VALUE;
  if (alpha == 0.f) k = 0;
  if (k > 0) {
    const int a_rows = ta ? k : m, b_rows = tb ? n : k;
    if (A == nullptr || B == nullptr || lda < (a_rows > 1 ? a_rows : 1) ||
        ldb < (b_rows > 1 ? b_rows : 1))
      return RTAT_STATUS_INVALID_VALUE;
  }
  dim3 grid((m + ST - 1) / ST, (n + ST - 1) / ST);
  hipLaunchKernelGGL(sgemm_kernel, grid, dim3(256), 0, h->stream, ta ? 1 : 0, tb ? 1 : 0, m, n,
                     k, alpha, A, (long)lda, B, (long)ldb, beta, C, (long)ldc, tri);
  return launch_status();
}

rtat_status_t launch_strsm(rtat_native_handle* h, bool left, bool lower, bool trans, bool unit,
                           int m, int n, float alpha, const float* A, int lda, float* B,
                           int ldb) {
  if (m < 0 || n < 0 || ldb < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  const int na = left ? m : n;
  if (lda < (na > 1 ? na : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (A == nullptr || B == nullptr) return RTAT_STATUS_INVALID_VALUE;
  const int nrhs = left ? n : m;
  hipLaunchKernelGGL(strsm_kernel, dim3((nrhs + 255) / 256), dim3(256), 0, h->stream,
                     left ? 1 : 0, lower ? 1 : 0, trans ? 1 : 0, unit ? 1 : 0, m, n, alpha, A,
                     (long)lda, B, (long)ldb);
  return launch_status();
}

}  // namespace rtat_native
