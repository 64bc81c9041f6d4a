// Bandwidth-bound kernels behind rtat_dgeam / rtat_sgeam / rtat_dfill / rtat_sfill:
// copy, re-stride (pad / unpad), scale, transpose through an LDS tile, accumulate, fill.
//
// These serve the reference's MatrixMove (src/matrix_ops/matrixop.h:307-344: B = alpha*op(A)
// into fresh scratch, beta = 0), MatrixAccumulate (matrixop.h:256-305: B = alpha*op(A) +
// beta*B in place on the caller's output) and the zero fill of MatrixSyrkAlloc
// (matrixop.h:612), all of which the reference routes through hipblasDgeam.
//
// Algorithmic traffic per call: (1 + [beta != 0]) reads + 1 write of the logical m x n.
#include "common.h"

#include <type_traits>

namespace rtat_native {

enum GeamMode { GEAM_ZERO = 0, GEAM_COPY = 1, GEAM_SCALE = 2, GEAM_AXPBY = 3 };

template <typename T>
__device__ inline T fused(T x, T y, T z);
template <>
__device__ inline double fused(double x, double y, double z) { return fma(x, y, z); }
template <>
__device__ inline float fused(float x, float y, float z) { return fmaf(x, y, z); }

// alpha*a + beta*b with one rounding for the sum: exact-product cases (alpha = 1 or beta a
// power of two) are then correctly rounded, which is what the bit-exact accumulate tests need.
template <typename T>
__device__ inline T combine(int mode, T alpha, T a, T beta, T b) {
  switch (mode) {
    case GEAM_COPY: return a;
    case GEAM_SCALE: return alpha * a;
    case GEAM_AXPBY: return fused<T>(beta, b, alpha * a);
    default: return T(0);
  }
}

template <typename T, int VEC>
struct VecOf;
template <> struct VecOf<double, 1> { typedef double type; };
template <> struct VecOf<double, 2> { typedef double type __attribute__((ext_vector_type(2))); };
template <> struct VecOf<float, 1> { typedef float type; };
template <> struct VecOf<float, 2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct VecOf<float, 4> { typedef float type __attribute__((ext_vector_type(4))); };

constexpr int NN_RUNS = 8;  // runs of 256 lanes per workgroup pass in the non-transposed kernel

// Streaming accesses: the data is touched once, so keep it from displacing anything in L2.
template <bool STREAM, typename T>
__device__ inline T stream_load(const T* p) {
  if constexpr (STREAM) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool STREAM, typename T>
__device__ inline void stream_store(T v, T* p) {
  if constexpr (STREAM) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// `valid` (<= VEC) consecutive elements at p; one vector access when all VEC are valid.
template <typename T, int VEC, bool STREAM>
__device__ inline void load_run(const T* p, int valid, T (&out)[VEC]) {
  if constexpr (VEC > 1) {
    if (valid == VEC) {
      typename VecOf<T, VEC>::type v =
          stream_load<STREAM>(reinterpret_cast<const typename VecOf<T, VEC>::type*>(p));
#pragma unroll
      for (int e = 0; e < VEC; ++e) out[e] = v[e];
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e)
    if (e < valid) out[e] = stream_load<STREAM>(p + e);
}

template <typename T, int VEC, bool STREAM>
__device__ inline void store_run(T* p, int valid, const T (&in)[VEC]) {
  if constexpr (VEC > 1) {
    if (valid == VEC) {
      typename VecOf<T, VEC>::type v;
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = in[e];
      stream_store<STREAM>(v, reinterpret_cast<typename VecOf<T, VEC>::type*>(p));
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e)
    if (e < valid) stream_store<STREAM>(in[e], p + e);
}

// C = alpha*A + beta*B, neither operand transposed.  One workgroup pass covers NN_RUNS runs
// of 256*VEC rows: RC consecutive runs down each of NN_RUNS / RC neighbouring columns; every
// lane issues all its loads before its first store.  Tall matrices take RC = NN_RUNS (one
// long contiguous stretch of a column per pass), short ones RC = 1.  VEC > 1 needs 16-byte
// aligned pointers and leading dimensions that keep columns aligned.  C may alias A or B:
// every element is read and written by the same lane.
template <typename T, int VEC, bool STREAM, int RC>
__global__ __launch_bounds__(256) void geam_nn_kernel(int m, int n, int mode, T alpha,
                                                     const T* A, long lda, T beta,
                                                     const T* B, long ldb, T* C, long ldc) {
  constexpr int CC = NN_RUNS / RC;
  const int row0 = (blockIdx.x * RC * 256 + threadIdx.x) * VEC;
  if (row0 >= m) return;
  for (int j0 = blockIdx.y * CC; j0 < n; j0 += gridDim.y * CC) {
    T a[NN_RUNS][VEC], b[NN_RUNS][VEC];
#pragma unroll
    for (int q = 0; q < NN_RUNS; ++q) {
      const int j = j0 + q / RC, row = row0 + (q % RC) * 256 * VEC;
#pragma unroll
      for (int e = 0; e < VEC; ++e) { a[q][e] = T(0); b[q][e] = T(0); }
      if (j < n && row < m) {
        const int valid = (m - row < VEC) ? m - row : VEC;
        if (mode != GEAM_ZERO) load_run<T, VEC, STREAM>(A + row + (long)j * lda, valid, a[q]);
        if (mode == GEAM_AXPBY) load_run<T, VEC, STREAM>(B + row + (long)j * ldb, valid, b[q]);
      }
    }
#pragma unroll
    for (int q = 0; q < NN_RUNS; ++q) {
      const int j = j0 + q / RC, row = row0 + (q % RC) * 256 * VEC;
      if (j < n && row < m) {
        const int valid = (m - row < VEC) ? m - row : VEC;
        T v[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = combine<T>(mode, alpha, a[q][e], beta, b[q][e]);
        store_run<T, VEC, STREAM>(C + row + (long)j * ldc, valid, v);
      }
    }
  }
}

// C = 0.  Stores alone go fastest with little work per workgroup: one 16-byte store per lane
// and column, a workgroup per 256-lane run of rows (measured on MI355X, 512 MiB: 6.6 TB/s
// against 5.3 with eight stores per lane).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void zero_kernel(int m, int n, T* C, long ldc) {
  const int row = (blockIdx.x * 256 + threadIdx.x) * VEC;
  if (row >= m) return;
  const int valid = (m - row < VEC) ? m - row : VEC;
  T z[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) z[e] = T(0);
  for (int j = blockIdx.y; j < n; j += gridDim.y)
    store_run<T, VEC, false>(C + row + (long)j * ldc, valid, z);
}

// C(m x n) = alpha*A^T + beta*op(B), A stored n x m.  A block of TI rows x TJ columns of C
// is gathered from A along A's contiguous dimension (runs of TJ elements) into LDS (row
// stride TJ+1: conflict-free both ways) and written out along C's contiguous dimension in
// runs of TI elements, so both global streams are coalesced.  TI = 128, TJ = 32 measured
// best on MI355X: long (1 KiB) write runs matter more than long read runs.  Workgroup x runs
// along C's rows, so neighbouring workgroups write neighbouring runs.
//
// XCD_ROWS, for a C whose columns start inside 128-byte lines (odd leading dimension, offset
// base): a TI-row run then begins and ends inside a line, and every line on a tile boundary
// is written in two parts by two workgroups.  The grid is a multiple of 8 wide, workgroup x
// runs on XCD x % 8, and each XCD takes a contiguous eighth of the nti tile rows, so that both
// parts of such a line meet in one L2.  The same goes for read runs that split lines (A_NT
// false: A's lines are loaded to stay, and the tile next along A's columns, which the same
// XCD takes a few workgroups later, finds the shared line there).
//
// WIDE: a leading dimension so long that a lane's byte offset within a tile passes 4 GiB; the
// offsets are then 64 bits wide (one plain instantiation serves such calls).
//
// SKEW, the better answer to such a C when the traffic is large: the row tiles are shifted,
// column by column, onto C's 128-byte lines.  Column j of tile row ti covers rows
// ti * TI - sc(j) .. + TI - 1, where sc(j) is the distance of the column's first element from
// the line boundary before it, so every TI-row run a workgroup writes starts on a line and no
// line is shared between workgroups (only the ends of a column are partial).  The tile is
// gathered from a window of TI + LINE rows, each lane keeping the elements its workgroup owns.
// The grid is a multiple of 8 wide, so that the tiles next to each other along A's columns,
// which share the lines at the ends of their read runs when A's columns split lines too, run on
// one XCD.  Measured on MI355X (doubles, old -> new): 6151 x 10007 from lda = 10010 into
// ldc = 6151 4.74 -> 5.5 TB/s, 8192^2 into ldc = 8195 4.8 -> 5.1, into an aligned C three
// elements off a line 4.84 -> 5.8, 8191^2 5.2 -> 5.75, 12000 x 9000 into ldc = 12001 5.0 -> 5.46.
template <typename T, int TI, int TJ, bool TRANS_B, bool STREAM, bool XCD_ROWS,
          bool A_NT = STREAM, bool SKEW = false, bool WIDE = false>
__global__ __launch_bounds__(256) void geam_t_kernel(int m, int n, int mode, T alpha,
                                                    const T* __restrict__ A, long lda, T beta,
                                                    const T* B, long ldb, T* C, long ldc,
                                                    int nti, int deal) {
  constexpr int LINE = SKEW ? 128 / (int)sizeof(T) : 0;  // elements of a 128-byte line
  constexpr int WIN = TI + LINE;                         // rows of the gather window
  __shared__ T tile_a[WIN][TJ + 1];
  __shared__ T tile_b[TRANS_B ? TI : 1][TJ + 1];
  static_assert(!(SKEW && TRANS_B), "the shifted tiles serve an untransposed B only");
  constexpr int RSTEP = 256 / TJ, RN = (WIN + RSTEP - 1) / RSTEP;  // gather: rows per pass
  constexpr int WSTEP = 256 / TI, WN = TJ / WSTEP;  // scatter: columns of the tile per pass
  const int rx = threadIdx.x % TJ, ry = threadIdx.x / TJ;
  const int wx = threadIdx.x % TI, wy = threadIdx.x / TI;
  // Workgroup -> tiles.  Plain: tile row blockIdx.x, the column tiles blockIdx.y, + gridDim.y, ...
  // deal = G > 0 (a grid 8 wide, one x per XCD): the column tiles are dealt to the XCDs in
  // groups of G neighbours, XCD x taking groups x, x + 8, ...; item q = blockIdx.y, + gridDim.y,
  // ... of an XCD's list walks a group tile row by tile row, the group's G column tiles
  // fastest.  That is the mapping for a C of few tile rows, which the row-wise ones would leave
  // on nti of the 8 XCDs, and it keeps both kinds of neighbours that share lines on one XCD
  // and close in time: the column tiles of a group (the lines at the ends of their read runs,
  // when A's columns split lines) and consecutive tile rows (the window rows of shifted tiles).
  // The eight XCDs read neighbouring groups at a time, 8 * G * TJ contiguous elements of each
  // column of A.
  int ti = blockIdx.x;
  if constexpr (XCD_ROWS) ti = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  if (deal == 0 && ti >= nti) return;
  const int njt = (n + TJ - 1) / TJ;
  // Distance (in elements) of C's first element from the line boundary before it.
  const long c_off =
      SKEW ? (long)((reinterpret_cast<uintptr_t>(C) / sizeof(T)) % (LINE > 0 ? LINE : 1)) : 0;
  auto shift_of = [&](int j) -> int {  // sc(j)
    if constexpr (SKEW) return (int)((c_off + (long)j * ldc) % LINE);
    else return 0;
  };
  // Addresses are a workgroup-uniform base (scalar registers) plus a 32-bit byte offset per
  // lane, the same for every pass of a loop: one address register per lane instead of a 64-bit
  // pair per access in flight (128-148 VGPRs came down to 64-79, and the shifted-tile form
  // went from three to four workgroups per CU).  The launcher checks that the offsets fit.
  typedef std::conditional_t<WIDE, size_t, unsigned> off_t;
  auto at = [](auto* uniform_base, off_t byte_offset) {
    typedef std::remove_pointer_t<decltype(uniform_base)> E;
    typedef std::conditional_t<std::is_const_v<E>, const char, char> Byte;
    return reinterpret_cast<E*>(reinterpret_cast<Byte*>(uniform_base) + byte_offset);
  };
  const off_t es = (off_t)sizeof(T);
  const off_t a_lane = ((off_t)ry * (off_t)lda + (off_t)rx) * es;
  const off_t bt_lane = ((off_t)ry * (off_t)ldb + (off_t)rx) * es;
  for (int q = blockIdx.y;; q += gridDim.y) {
    int jt = q, jt_next = q + (int)gridDim.y;
    if (deal != 0) {
      const int per_group = nti * deal;
      const int group = (int)blockIdx.x + 8 * (q / per_group), rem = q % per_group;
      if (group * deal >= njt) break;  // past the XCD's last group
      ti = rem / deal;
      jt = group * deal + rem % deal;
      jt_next = 0;  // never the last pass: the barrier behind a tile is kept
      if (jt >= njt) continue;  // the last group may be short of column tiles
    }
    if (jt >= njt) break;
    const int i0 = ti * TI, j0 = jt * TJ;
    const T* a_tile = A + j0 + (long)(i0 - LINE) * lda;   // first element of the gather window
    const T* bt_tile = B + j0 + (long)i0 * ldb;           // (TRANS_B) the same of B
    T* c_tile = C + (i0 - LINE) + (long)j0 * ldc;         // LINE rows before the tile of C
    const T* b_tile = B + (i0 - LINE) + (long)j0 * ldb;
    const bool last_pass = jt_next >= njt;
    // WHOLE: the tile lies inside C, no per-element bounds.  COPY: alpha = 1 and no second
    // operand, the plain transpose: nothing of B is loaded, held or tested for.
    auto tile = [&](auto whole_tag, auto copy_tag) {
      constexpr bool WHOLE = decltype(whole_tag)::value;
      constexpr bool COPY = decltype(copy_tag)::value;
      T va[RN], vb[RN];
      const int sc_r = shift_of(j0 + rx);
#pragma unroll
      for (int s = 0; s < RN; ++s) {
        const int li = ry + s * RSTEP;  // row of the window; the window starts LINE rows early
        const int i = i0 - LINE + li;
        va[s] = T(0);
        vb[s] = T(0);
        bool wanted = WHOLE || (j0 + rx < n && i >= 0 && i < m);
        if constexpr (SKEW) wanted = wanted && li >= LINE - sc_r && li < LINE - sc_r + TI;
        if (RN * RSTEP != WIN) wanted = wanted && li < WIN;
        if (wanted) {
          va[s] = stream_load<A_NT>(at(a_tile + (long)(s * RSTEP) * lda, a_lane));
          if (!COPY && TRANS_B && mode == GEAM_AXPBY)
            vb[s] = stream_load<STREAM>(at(bt_tile + (long)(s * RSTEP) * ldb, bt_lane));
        }
      }
#pragma unroll
      for (int s = 0; s < RN; ++s) {
        const int li = ry + s * RSTEP;
        if (RN * RSTEP == WIN || li < WIN) {
          tile_a[li][rx] = va[s];
          if (!COPY && TRANS_B) tile_b[li][rx] = vb[s];
        }
      }
      __syncthreads();
      // Column wy + s * WSTEP of the tile, row wx less the column's shift: the lane's offset
      // from LINE rows above the column pair's first element (never negative).
      auto c_lane = [&](int s, long ld) {
        return (off_t)((long)wy * ld + wx + LINE - shift_of(j0 + wy + s * WSTEP)) * es;
      };
      T b[WN];
#pragma unroll
      for (int s = 0; s < WN; ++s) {
        const int j = wy + s * WSTEP;
        const int i = i0 - shift_of(j0 + j) + wx;
        b[s] = T(0);
        if (!COPY && !TRANS_B && mode == GEAM_AXPBY &&
            (WHOLE || (i >= 0 && i < m && j0 + j < n)))
          b[s] = stream_load<STREAM>(at(b_tile + (long)(s * WSTEP) * ldb, c_lane(s, ldb)));
      }
#pragma unroll
      for (int s = 0; s < WN; ++s) {
        const int j = wy + s * WSTEP;
        const int sc = shift_of(j0 + j);
        const int i = i0 - sc + wx;
        if (WHOLE || (i >= 0 && i < m && j0 + j < n)) {
          const T a = tile_a[LINE - sc + wx][j];
          const T bb = (!COPY && TRANS_B) ? tile_b[wx][j] : b[s];
          stream_store<STREAM>(COPY ? a : combine<T>(mode, alpha, a, beta, bb),
                               at(c_tile + (long)(s * WSTEP) * ldc, c_lane(s, ldc)));
        }
      }
      if (!last_pass) __syncthreads();  // the tile in LDS is free for the next pass
    };
    // A tile whose every column may be shifted by up to LINE - 1 rows lies inside C when the
    // rows from LINE before it to its last one do.
    const bool whole = i0 - LINE >= 0 && i0 + TI <= m && j0 + TJ <= n;
    if (mode == GEAM_COPY) {
      if (whole) tile(std::true_type{}, std::true_type{});
      else tile(std::false_type{}, std::true_type{});
    } else {
      if (whole) tile(std::true_type{}, std::false_type{});
      else tile(std::false_type{}, std::false_type{});
    }
  }
}

template <typename T>
__device__ inline T quiet_nan();
template <> __device__ inline double quiet_nan<double>() {
  return __longlong_as_double(0x7ff8000000000000ll);
}
template <> __device__ inline float quiet_nan<float>() { return __int_as_float(0x7fc00000); }

// Synthetic operand: element (i, j) from the counter-based generator, padding rows = NaN.
template <typename T>
__global__ __launch_bounds__(256) void fill_kernel(T* A, int m, int n, long ld, uint64_t seed,
                                                  int kind) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= ld) return;
  for (int j = blockIdx.y; j < n; j += gridDim.y) {
    T v;
    if (i >= m) {
      v = quiet_nan<T>();
    } else if (kind == RTAT_FILL_SYMMETRIC) {
      const uint32_t hi = (uint32_t)(i > j ? i : j), lo = (uint32_t)(i > j ? j : i);
      v = (T)(2.0 * unit_uniform(seed, hi, lo) - 1.0);
    } else if (kind == RTAT_FILL_TRI_LOWER) {
      const double u = unit_uniform(seed, (uint32_t)i, (uint32_t)j);
      if (i > j) v = (T)((2.0 * u - 1.0) / (double)m);
      else if (i == j) v = (T)(1.0 + u);
      else v = quiet_nan<T>();
    } else if (kind == RTAT_FILL_TRI_FULL) {
      const uint32_t hi = (uint32_t)(i > j ? i : j), lo = (uint32_t)(i > j ? j : i);
      const double u = unit_uniform(seed, hi, lo);
      v = (i == j) ? (T)(1.0 + u) : (T)((2.0 * u - 1.0) / (double)m);
    } else if (kind == RTAT_FILL_UNIT_INTERVAL) {
      v = (T)(1.0 - unit_uniform(seed, (uint32_t)i, (uint32_t)j));
    } else {
      v = (T)(2.0 * unit_uniform(seed, (uint32_t)i, (uint32_t)j) - 1.0);
    }
    A[i + (long)j * ld] = v;
  }
}

// ---- two moves in one launch ---------------------------------------------------------------
// C_i = op_i(A_i), i = 0, 1: the copies / transposes / pad copies a variant makes of both GEMM
// operands before the multiply (reference src/methods/gemm.cpp:98-106 builds them as two
// MatrixMove nodes, two geam launches).  The workgroups of one launch are dealt to the two jobs;
// an untransposed job moves 256 * VEC rows of 8 neighbouring columns per workgroup (all loads
// before the first store, as geam_nn_kernel does), a transposed one a 128 x 32 tile through LDS
// (as geam_t_kernel does).  One launch instead of two saves the gap between them, which is
// what a small problem's variant pays for most.
template <typename T>
struct MoveJob {
  const T* A;
  T* C;
  long lda, ldc;
  int m, n;        // shape of C
  int trans;       // C = A^T (A stored n x m)
  int vec;         // untransposed: elements per access (16 bytes' worth, or 1)
  unsigned tiles_x, blocks;
};

template <typename T, bool STREAM>
__global__ __launch_bounds__(256) void move_pair_kernel(MoveJob<T> j0, MoveJob<T> j1) {
  constexpr int TI = 128, TJ = 32, CC = 8, VMAX = 16 / (int)sizeof(T);
  __shared__ T tile[TI][TJ + 1];
  const bool second = blockIdx.x >= j0.blocks;
  const MoveJob<T>& job = second ? j1 : j0;
  const unsigned b = second ? blockIdx.x - j0.blocks : blockIdx.x;
  const int bx = (int)(b % job.tiles_x), by = (int)(b / job.tiles_x);
  if (!job.trans) {
    auto rows = [&](auto vtag) {
      constexpr int V = decltype(vtag)::value;
      const int row = (bx * 256 + (int)threadIdx.x) * V;
      if (row >= job.m) return;
      const int valid = (job.m - row < V) ? job.m - row : V;
      T v[CC][V];
#pragma unroll
      for (int q = 0; q < CC; ++q) {
        const int j = by * CC + q;
        if (j < job.n) load_run<T, V, STREAM>(job.A + row + (long)j * job.lda, valid, v[q]);
      }
#pragma unroll
      for (int q = 0; q < CC; ++q) {
        const int j = by * CC + q;
        if (j < job.n) store_run<T, V, STREAM>(job.C + row + (long)j * job.ldc, valid, v[q]);
      }
    };
    if (job.vec > 1) rows(std::integral_constant<int, VMAX>{});
    else rows(std::integral_constant<int, 1>{});
    return;
  }
  constexpr int RSTEP = 256 / TJ, RN = TI / RSTEP, WSTEP = 256 / TI, WN = TJ / WSTEP;
  const int rx = threadIdx.x % TJ, ry = threadIdx.x / TJ;
  const int wx = threadIdx.x % TI, wy = threadIdx.x / TI;
  const int i0 = bx * TI, j0c = by * TJ;
  T va[RN];
#pragma unroll
  for (int s = 0; s < RN; ++s) {
    const int i = i0 + ry + s * RSTEP;
    va[s] = T(0);
    if (j0c + rx < job.n && i < job.m)
      va[s] = stream_load<STREAM>(job.A + (j0c + rx) + (long)i * job.lda);
  }
#pragma unroll
  for (int s = 0; s < RN; ++s) tile[ry + s * RSTEP][rx] = va[s];
  __syncthreads();
#pragma unroll
  for (int s = 0; s < WN; ++s) {
    const int j = wy + s * WSTEP;
    if (i0 + wx < job.m && j0c + j < job.n)
      stream_store<STREAM>(tile[wx][j], job.C + (i0 + wx) + (long)(j0c + j) * job.ldc);
  }
}

static inline bool move_aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

template <typename T>
rtat_status_t launch_move_pair(rtat_native_handle* h, const rtat_move_t* first,
                               const rtat_move_t* second) {
  const rtat_move_t* in[2] = {first, second};
  MoveJob<T> job[2];
  size_t bytes = 0;
  for (int q = 0; q < 2; ++q) {
    const rtat_move_t& mv = *in[q];
    if (mv.trans != RTAT_OP_N && mv.trans != RTAT_OP_T) return RTAT_STATUS_INVALID_ENUM;
    const bool t = mv.trans == RTAT_OP_T;
    if (mv.m < 0 || mv.n < 0 || mv.ldc < (mv.m > 1 ? mv.m : 1) ||
        mv.lda < ((t ? mv.n : mv.m) > 1 ? (t ? mv.n : mv.m) : 1))
      return RTAT_STATUS_INVALID_VALUE;
    const bool empty = mv.m == 0 || mv.n == 0;
    if (!empty && (mv.A == nullptr || mv.C == nullptr || mv.A == mv.C))
      return RTAT_STATUS_INVALID_VALUE;
    MoveJob<T>& j = job[q];
    j.A = static_cast<const T*>(mv.A);
    j.C = static_cast<T*>(mv.C);
    j.lda = mv.lda;
    j.ldc = mv.ldc;
    j.m = mv.m;
    j.n = mv.n;
    j.trans = t ? 1 : 0;
    constexpr int VMAX = 16 / (int)sizeof(T);
    j.vec = (!t && move_aligned16(mv.A) && move_aligned16(mv.C) && mv.lda % VMAX == 0 &&
             mv.ldc % VMAX == 0) ? VMAX : 1;
    if (empty) {
      j.tiles_x = 1;
      j.blocks = 0;
    } else if (t) {
      j.tiles_x = (unsigned)((mv.m + 127) / 128);
      j.blocks = j.tiles_x * (unsigned)((mv.n + 31) / 32);
    } else {
      j.tiles_x = (unsigned)((mv.m + 256 * j.vec - 1) / (256 * j.vec));
      j.blocks = j.tiles_x * (unsigned)((mv.n + 7) / 8);
    }
    if ((size_t)j.tiles_x * (size_t)((t ? (mv.n + 31) / 32 : (mv.n + 7) / 8) + 1) > 0x3fffffffu)
      return RTAT_STATUS_INVALID_VALUE;
    bytes += 2 * (size_t)mv.m * (size_t)mv.n * sizeof(T);
  }
  const unsigned grid = job[0].blocks + job[1].blocks;
  if (grid == 0) return RTAT_STATUS_SUCCESS;
  // Non-temporal accesses from the traffic on at which the single-job kernels switch.
  if (bytes > ((size_t)288 << 20))
    hipLaunchKernelGGL((move_pair_kernel<T, true>), dim3(grid), dim3(256), 0, h->stream, job[0],
                       job[1]);
  else
    hipLaunchKernelGGL((move_pair_kernel<T, false>), dim3(grid), dim3(256), 0, h->stream, job[0],
                       job[1]);
  return launch_status();
}
template rtat_status_t launch_move_pair<double>(rtat_native_handle*, const rtat_move_t*,
                                                const rtat_move_t*);
template rtat_status_t launch_move_pair<float>(rtat_native_handle*, const rtat_move_t*,
                                               const rtat_move_t*);

// ---- streaming probes ---------------------------------------------------------------------
// What the memory system delivers to a kernel that does nothing but stream: the yardstick
// the copy / transpose figures are read against.  16-byte non-temporal accesses, 256 lanes,
// U accesses per lane in flight; the shapes are the fastest of a sweep over U, workgroup
// size, grid and cache policy on MI355X (read U = 8, write U = 1, copy U = 8).
typedef double probe_vec_t __attribute__((ext_vector_type(2)));
constexpr int PROBE_U = 8;
constexpr size_t PROBE_GRAIN = (size_t)256 * 16 * PROBE_U;  // bytes per workgroup

__global__ __launch_bounds__(256) void probe_read_kernel(const probe_vec_t* __restrict__ in,
                                                        double* sink) {
  const probe_vec_t* q = in + (size_t)blockIdx.x * 256 * PROBE_U + threadIdx.x;
  probe_vec_t v[PROBE_U];
#pragma unroll
  for (int u = 0; u < PROBE_U; ++u) v[u] = __builtin_nontemporal_load(q + (size_t)u * 256);
  probe_vec_t acc = v[0];
#pragma unroll
  for (int u = 1; u < PROBE_U; ++u) acc += v[u];
  // Never true for finite data; keeps the loads alive without a store per lane.
  if (acc[0] + acc[1] == __longlong_as_double(0x7ff0000000000000ll)) sink[threadIdx.x] = acc[0];
}

__global__ __launch_bounds__(256) void probe_write_kernel(probe_vec_t* __restrict__ out) {
  const probe_vec_t v = {1.0, 2.0};
  __builtin_nontemporal_store(v, out + (size_t)blockIdx.x * 256 + threadIdx.x);
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const probe_vec_t* __restrict__ in,
                                                        probe_vec_t* __restrict__ out) {
  const size_t base = (size_t)blockIdx.x * 256 * PROBE_U + threadIdx.x;
  probe_vec_t v[PROBE_U];
#pragma unroll
  for (int u = 0; u < PROBE_U; ++u) v[u] = __builtin_nontemporal_load(in + base + (size_t)u * 256);
#pragma unroll
  for (int u = 0; u < PROBE_U; ++u) __builtin_nontemporal_store(v[u], out + base + (size_t)u * 256);
}

rtat_status_t launch_probe(rtat_native_handle* h, int kind, const void* src, void* dst,
                           size_t bytes) {
  if (kind < RTAT_PROBE_READ || kind > RTAT_PROBE_COPY) return RTAT_STATUS_INVALID_ENUM;
  if (bytes % PROBE_GRAIN != 0 || bytes / 4096 > 0x7fffffffu) return RTAT_STATUS_INVALID_VALUE;
  if (bytes == 0) return RTAT_STATUS_SUCCESS;
  const bool reads = kind != RTAT_PROBE_WRITE;
  if ((reads && (src == nullptr || (reinterpret_cast<uintptr_t>(src) & 15u))) || dst == nullptr ||
      (reinterpret_cast<uintptr_t>(dst) & 15u))
    return RTAT_STATUS_INVALID_VALUE;
  if (kind == RTAT_PROBE_READ) {
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)(bytes / PROBE_GRAIN)), dim3(256), 0,
                       h->stream, static_cast<const probe_vec_t*>(src), static_cast<double*>(dst));
  } else if (kind == RTAT_PROBE_WRITE) {
    hipLaunchKernelGGL(probe_write_kernel, dim3((unsigned)(bytes / 4096)), dim3(256), 0, h->stream,
                       static_cast<probe_vec_t*>(dst));
  } else {
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)(bytes / PROBE_GRAIN)), dim3(256), 0,
                       h->stream, static_cast<const probe_vec_t*>(src),
                       static_cast<probe_vec_t*>(dst));
  }
  return launch_status();
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T>
rtat_status_t launch_geam(rtat_native_handle* h, bool ta, bool tb, int m, int n, T alpha,
                          const T* A, int lda, T beta, const T* B, int ldb, T* C, int ldc) {
  if (m < 0 || n < 0 || ldc < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  bool use_a = alpha != T(0), use_b = beta != T(0);
  // Single-operand forms are expressed on the A slot.
  if (!use_a && use_b) {
    A = B; lda = ldb; ta = tb; alpha = beta; beta = T(0);
    use_a = true; use_b = false;
  }
  if (use_a && (A == nullptr || lda < (ta ? n : m) || lda < 1)) return RTAT_STATUS_INVALID_VALUE;
  if (use_b && (B == nullptr || ldb < (tb ? n : m) || ldb < 1)) return RTAT_STATUS_INVALID_VALUE;
  if (C == nullptr) return RTAT_STATUS_INVALID_VALUE;
  // hipBLAS in-place rules: an aliased operand must be untransposed with equal ld.
  if (use_a && (const T*)C == A && (ta || lda != ldc)) return RTAT_STATUS_INVALID_VALUE;
  if (use_b && (const T*)C == B && (tb || ldb != ldc)) return RTAT_STATUS_INVALID_VALUE;

  int mode = GEAM_ZERO;
  if (use_a && use_b) mode = GEAM_AXPBY;
  else if (use_a) mode = (alpha == T(1)) ? GEAM_COPY : GEAM_SCALE;
  if (mode == GEAM_ZERO) { ta = false; tb = false; }
  if (mode != GEAM_AXPBY) tb = false;
  // Put the transposed operand (if only one) on the A slot: the sum is symmetric.
  if (!ta && tb) {
    const T* p = A; A = B; B = p;
    int l = lda; lda = ldb; ldb = l;
    T s = alpha; alpha = beta; beta = s;
    ta = true; tb = false;
  }

  hipStream_t st = h->stream;
  // Traffic beyond the 256 MiB last-level cache is moved with non-temporal accesses.
  // Measured on MI355X (doubles, square, the same call repeated): copies and transposes
  // gain from 324 MiB of traffic on (n = 4608: transpose 5.03 -> 5.57 TB/s, n = 8192: 4.77 ->
  // 5.81) and lose at 256 MiB (n = 4096: 6.14 -> 5.37); accumulates gain from 600 MiB on
  // (n = 5120: 5.32 -> 5.98) and lose at 486 MiB; zero fills lose up to 512 MiB at least.
  const size_t passes = mode == GEAM_ZERO ? 1 : mode == GEAM_AXPBY ? 3 : 2;
  const size_t threshold = passes == 2 ? (size_t)288 << 20 : (size_t)512 << 20;
  const bool stream = passes * (size_t)m * (size_t)n * sizeof(T) > threshold;
  if (!ta) {
    constexpr int VMAX = 16 / sizeof(T);  // elements of a 16-byte access
    const bool vec_ok = aligned16(C) && (ldc % VMAX == 0) &&
                        (mode == GEAM_ZERO || (aligned16(A) && lda % VMAX == 0)) &&
                        (mode != GEAM_AXPBY || (aligned16(B) && ldb % VMAX == 0));
    // Shape of a workgroup pass: rc consecutive runs (of 256 lanes) down each of NN_RUNS / rc
    // neighbouring columns.  Measured on MI355X (doubles, sixteen shapes from 1000 x 30000 to
    // 16384^2): copies and fills of columns up to 96 KiB move fastest in long stretches, as
    // long as the stretches divide the column evenly - a workgroup left with part of a
    // stretch keeps its slot as long as a full one (4608^2 as 8 + 1 runs 4.91 TB/s, as nine
    // single runs 5.95; 6144^2 as 8 + 4 runs 5.46, as three times 4 runs 6.21; 10007 x 6151
    // 5.98 -> 6.17): rc is the largest of 8, 4, 2, 1 that wastes the fewest runs.  Longer
    // columns are 2-7 % faster as single runs; the accumulate gains with one and loses with
    // another leading dimension, and stays with single runs.
    const int vec = vec_ok ? VMAX : 1;
    // Zero fill of columns that start on 4 KiB boundaries: one store per lane (8192^2 5.3 ->
    // 6.6 TB/s, 16384^2 6.2 -> 6.8); columns that start elsewhere do better in the long
    // stretches below (ld = 8224: 5.5 against 5.0; odd ld: 4.9 against 3.9).
    if (mode == GEAM_ZERO && vec_ok && ((size_t)ldc * sizeof(T)) % 4096 == 0 &&
        (reinterpret_cast<uintptr_t>(C) % 4096) == 0) {
      dim3 zgrid((m + 256 * VMAX - 1) / (256 * VMAX), (unsigned)(n > 65535 ? 65535 : n));
      hipLaunchKernelGGL((zero_kernel<T, VMAX>), zgrid, dim3(256), 0, st, m, n, C, (long)ldc);
      return launch_status();
    }
    int rc = 1;
    if (mode != GEAM_AXPBY && (size_t)m * sizeof(T) <= ((size_t)96 << 10)) {
      const int runs = (m + 256 * vec - 1) / (256 * vec);
      int least = runs * NN_RUNS;
      for (int r = NN_RUNS; r >= 1; r /= 2) {
        const int waste = (runs + r - 1) / r * r - runs;
        if (waste < least) { least = waste; rc = r; }
      }
    }
    const int cc = NN_RUNS / rc;
    dim3 grid((m + 256 * vec * rc - 1) / (256 * vec * rc), (unsigned)((n + cc - 1) / cc));
    if (grid.y > 65535u) grid.y = 65535u;
    auto launch = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, m, n, mode, alpha, A, (long)lda, beta, B,
                         (long)ldb, C, (long)ldc);
    };
    auto by_rc = [&](auto vtag, auto stag) {
      constexpr int V = decltype(vtag)::value;
      constexpr bool S = decltype(stag)::value;
      if (rc == 8) launch(geam_nn_kernel<T, V, S, 8>);
      else if (rc == 4) launch(geam_nn_kernel<T, V, S, 4>);
      else if (rc == 2) launch(geam_nn_kernel<T, V, S, 2>);
      else launch(geam_nn_kernel<T, V, S, 1>);
    };
    if (vec_ok) {
      if (stream) by_rc(std::integral_constant<int, VMAX>{}, std::true_type{});
      else by_rc(std::integral_constant<int, VMAX>{}, std::false_type{});
    } else {
      if (stream) by_rc(std::integral_constant<int, 1>{}, std::true_type{});
      else by_rc(std::integral_constant<int, 1>{}, std::false_type{});
    }
  } else if (!tb) {
    constexpr int TI = 128, TJ = 32, LINE = 128 / (int)sizeof(T);
    // Columns of C that start inside a 128-byte line (odd leading dimension, offset base):
    // lines on tile boundaries are written in two parts by two workgroups, and each XCD takes
    // a contiguous eighth of the tile rows so that both parts meet in one L2.  Measured on
    // MI355X, doubles: 8192^2 into ldc = 8195 4.35 -> 4.8 TB/s, 6151 x 10007 into ldc = 6151
    // 4.2 -> 4.6, 65539 x 256 4.73 -> 5.19, accumulates 4.65-5.1 -> 4.97-5.4.
    // Columns of A that start inside a line: a read run shares its first and last line with
    // the tiles next along A's columns.  The same mapping runs those on one XCD a few
    // workgroups apart, and A is loaded to stay, so that the second finds the line in L2
    // (6151 x 10007 from lda = 10010: 4.59 -> 4.76, 8192^2 from lda = 8194 into 8194: 5.11 ->
    // 5.34; into aligned columns 8192^2 from lda = 8195 5.64 -> 5.80, its accumulate 6.03 ->
    // 6.39, 65536 x 600 from lda = 603 4.62 -> 5.72); either measure alone gains nothing.
    const bool split_lines =
        (reinterpret_cast<uintptr_t>(C) / sizeof(T)) % LINE != 0 || ldc % LINE != 0;
    const bool split_reads =
        (reinterpret_cast<uintptr_t>(A) / sizeof(T)) % LINE != 0 || lda % LINE != 0;
    // Large traffic into such a C: row tiles shifted onto C's lines (SKEW), one more tile row
    // for the rows the shift moves past the last whole tile.
    const bool skew = split_lines && stream;
    dim3 grid((m + (skew ? LINE - 1 : 0) + TI - 1) / TI, (unsigned)((n + TJ - 1) / TJ));
    if (grid.y > 65535u) grid.y = 65535u;
    const int nti = (int)grid.x;
    // The mappings that keep line-sharing tiles on one XCD deal whole tile rows to the XCDs:
    // with few tile rows (or a count just past a multiple of 8) some XCDs get little or
    // nothing - a C of 100 rows ran on one XCD, at 1.3 TB/s.  Then the column tiles are dealt
    // instead (see the kernel), if they divide more evenly.
    // Groups of 8 measured best on MI355X (doubles, 1 -> 8): 8192^2 into ldc = 8195 4.99 ->
    // 5.72 TB/s with 21 % less fetched, 4099 x 6151 from lda = 6154 into ldc = 4099 5.67 -> 6.54,
    // 6151 x 10007 from lda = 10010 into ldc = 6151 level at 5.4 with 20 % less fetched (30 %
    // more than the algorithmic bytes came down to 4 %).
    constexpr int DEAL_GROUP = 8;
    int deal = 0;
    if (split_lines || split_reads) {
      const long njt = (n + TJ - 1) / TJ, groups = (njt + DEAL_GROUP - 1) / DEAL_GROUP;
      const double by_rows = (double)nti / (double)((nti + 7) / 8 * 8);
      const double by_cols = (double)njt / (double)((njt + 7) / 8 * 8);
      if (by_cols > by_rows) {
        deal = DEAL_GROUP;
        const long items = (long)nti * DEAL_GROUP * ((groups + 7) / 8);
        grid = dim3(8, (unsigned)(items > 65535 ? 65535 : items));
      } else {
        grid.x = (grid.x + 7) / 8 * 8;
      }
    }
    auto launch = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, dim3(256), 0, st, m, n, mode, alpha, A, (long)lda, beta, B,
                         (long)ldb, C, (long)ldc, nti, deal);
    };
    // A lane's byte offset within a tile: up to 8 columns of A, 2 of B or C.
    const bool wide = 8 * (size_t)lda * sizeof(T) >= ((size_t)1 << 32) ||
                      2 * (size_t)ldc * sizeof(T) >= ((size_t)1 << 32) ||
                      (mode == GEAM_AXPBY && 2 * (size_t)ldb * sizeof(T) >= ((size_t)1 << 32));
    if (wide) {
      dim3 plain((unsigned)((m + TI - 1) / TI), (unsigned)((n + TJ - 1) / TJ));
      if (plain.y > 65535u) plain.y = 65535u;
      hipLaunchKernelGGL((geam_t_kernel<T, TI, TJ, false, false, false, false, false, true>),
                         plain, dim3(256), 0, st, m, n, mode, alpha, A, (long)lda, beta, B,
                         (long)ldb, C, (long)ldc, (int)plain.x, 0);
    } else if (skew) {
      if (split_reads) launch(geam_t_kernel<T, TI, TJ, false, true, false, false, true>);
      else launch(geam_t_kernel<T, TI, TJ, false, true, false, true, true>);
    } else if (split_lines || split_reads) {
      if (stream && split_reads) launch(geam_t_kernel<T, TI, TJ, false, true, true, false>);
      else if (stream) launch(geam_t_kernel<T, TI, TJ, false, true, true>);
      else launch(geam_t_kernel<T, TI, TJ, false, false, true>);
    } else {
      if (stream) launch(geam_t_kernel<T, TI, TJ, false, true, false>);
      else launch(geam_t_kernel<T, TI, TJ, false, false, false>);
    }
  } else {
    constexpr int TILE = 32;
    dim3 grid((m + TILE - 1) / TILE, (unsigned)((n + TILE - 1) / TILE));
    if (grid.y > 65535u) grid.y = 65535u;
    const bool wide = 8 * (size_t)lda * sizeof(T) >= ((size_t)1 << 32) ||
                      8 * (size_t)ldb * sizeof(T) >= ((size_t)1 << 32) ||
                      8 * (size_t)ldc * sizeof(T) >= ((size_t)1 << 32);
    if (wide)
      hipLaunchKernelGGL((geam_t_kernel<T, TILE, TILE, true, false, false, false, false, true>), grid,
                         dim3(256), 0, st, m, n, mode, alpha, A, (long)lda, beta, B, (long)ldb, C,
                         (long)ldc, (int)grid.x, 0);
    else
      hipLaunchKernelGGL((geam_t_kernel<T, TILE, TILE, true, false, false>), grid, dim3(256), 0, st,
                         m, n, mode, alpha, A, (long)lda, beta, B, (long)ldb, C, (long)ldc,
                         (int)grid.x, 0);
  }
  return launch_status();
}

template <typename T>
rtat_status_t launch_fill(rtat_native_handle* h, T* A, int m, int n, int ld, uint64_t seed,
                          int kind) {
  if (m < 0 || n < 0 || ld < (m > 1 ? m : 1) || kind < 0 || kind > RTAT_FILL_TRI_FULL)
    return RTAT_STATUS_INVALID_VALUE;
  if ((kind == RTAT_FILL_SYMMETRIC || kind == RTAT_FILL_TRI_LOWER || kind == RTAT_FILL_TRI_FULL) &&
      m != n)
    return RTAT_STATUS_INVALID_VALUE;
  if (n == 0 || ld == 0) return RTAT_STATUS_SUCCESS;
  if (A == nullptr) return RTAT_STATUS_INVALID_VALUE;
  dim3 grid((ld + 255) / 256, (unsigned)(n > 65535 ? 65535 : n));
  hipLaunchKernelGGL((fill_kernel<T>), grid, dim3(256), 0, h->stream, A, m, n, (long)ld, seed,
                     kind);
  return launch_status();
}

template rtat_status_t launch_geam<double>(rtat_native_handle*, bool, bool, int, int, double,
                                           const double*, int, double, const double*, int,
                                           double*, int);
template rtat_status_t launch_geam<float>(rtat_native_handle*, bool, bool, int, int, float,
                                          const float*, int, float, const float*, int, float*,
                                          int);
template rtat_status_t launch_fill<double>(rtat_native_handle*, double*, int, int, int, uint64_t,
                                           int);
template rtat_status_t launch_fill<float>(rtat_native_handle*, float*, int, int, int, uint64_t,
                                          int);

}  // namespace rtat_native
