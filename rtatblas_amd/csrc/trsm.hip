// Blocked triangular solve for gfx950 (double and float from one template).
//
// Serves gpuTtrsm of the reference (src/matrix_ops/matrixop.h:78-109), which forwards to
// hipblas{D,S}trsm: solve op(A) X = alpha B (left) or X op(A) = alpha B (right) in place in B.
//
// Method
//   1. The NB x NB diagonal blocks of A (NB = 128) are inverted, one workgroup per block,
//      entirely in LDS (trtri_kernel), into scratch.
//   2. The solve recurses on halves of the triangular dimension: solve one half, update the
//      other with one large-k GEMM (alpha = -1, beta = 1) on the MFMA core, solve the other
//      half.
//   3. A range of at most one panel (512 or 1024 rows) of the triangular dimension is solved by one
//      launch of trsm_panel_kernel: right-hand sides are independent, so each workgroup takes
//      a slab of 16 of them, keeps the slab's panel rows in LDS and runs the whole blocked
//      substitution on it (X_i = inv(M_ii) B_i, B_j -= M_ji X_i for the blocks of the panel)
//      with MFMAs.  The blocks of M it needs (the inverses and the off-diagonal blocks inside
//      each panel) are laid out once per call, by the launch that inverts the diagonal
//      blocks, as 128 x 128 column-major blocks of M in scratch; all workgroups read them, so
//      they live in L2.
//      With more right-hand sides than one such slab per CU, 512-row panels go to
//      trsm_panel_wide_kernel instead: 32 right-hand sides per workgroup, the slab held in
//      registers, half the traffic from L2 for the blocks of M, which the first launch then
//      lays out in the order the lanes of that kernel consume them.
//   All sixteen side / uplo / trans / diag combinations run natively and alike: a right-hand
//   solve is the left-hand solve of the transposed system (the slab is loaded and stored
//   transposed, M = op(A)^T), trans flips the effective triangle, inv(op(T)) = op(inv(T)).
//
// Flop count used for reporting: m*m*n (left), m*n*n (right).
#include "common.h"
#include "mfma.h"

namespace rtat_native {

constexpr int TRTRI_LD = NB + 1;  // odd stride: a row walk and a column walk are both conflict free
constexpr int TRTRI_THREADS = 256;
constexpr int TRTRI_SB = 16;      // diagonal sub-blocks inverted by substitution
constexpr int TRTRI_PACK_EACH = 4;  // off-diagonal blocks laid out by one packing workgroup
constexpr size_t TRTRI_LDS_ELEMS = (size_t)(NB * TRTRI_LD + 3 * NB);

// Fragment order of a 128 x 128 block of M for the 16x16x4 MFMAs of trsm_panel_wide_kernel: wave
// v = row / 16 of a workgroup takes MFMA step group g = k / 4E (E = elements per 16 bytes) with
// one 16-byte load per lane, lane = 16 kq + row % 16 holding k = 4E g + E kq + e, e = 0 .. E-1;
// the 64 lanes' loads of one group are 1 KiB in a row.
template <class T>
__host__ __device__ inline int frag_offset(int row, int k) {
  constexpr int E = Elem<T>::E, NGRP = NB / (4 * E);
  const int v = row >> 4, r16 = row & 15, g = k / (4 * E), kq = (k % (4 * E)) / E, e = k % E;
  return ((v * NGRP + g) * 64 + 16 * kq + r16) * E + e;
}
template <class T>
__host__ __device__ inline int block_offset(int row, int k, int frag) {
  return frag ? frag_offset<T>(row, k) : row + k * NB;
}

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
//
// The same launch also packs, for the panel solve, the off-diagonal 128 x 128 blocks of every
// diagonal panel (panel_blocks blocks square) of the system matrix M = op'(A) (workgroups past the diagonal
// blocks): M's block in M's own orientation, zero past the end of A, so that the panel kernel
// reads every block the same way whatever the transposition, alignment and raggedness of A.
// The inverses are written in M's orientation too (inv(T^T) = inv(T)^T).
// Both kinds of block are written column-major, element (r, k) at r + 128 k, or (frag != 0) in
// the order trsm_panel_wide_kernel's lanes consume them (frag_offset).
template <class T>
__global__ __launch_bounds__(TRTRI_THREADS) void trtri_kernel(const T* A, long lda, int na, int lower,
                                                             int unit, int mtrans, T* out,
                                                             T* packed, int panel_blocks, int frag) {
  extern __shared__ __align__(16) unsigned char sm_raw[];
  T* sm = reinterpret_cast<T*>(sm_raw);
  constexpr int LD = TRTRI_LD, SB = TRTRI_SB;
  T* L = sm;                 // NB x NB, column-major, ld = LD
  T* col = sm + NB * LD;     // 2 x NB column hand-over
  T* dinv = col + 2 * NB;    // reciprocals of the diagonal
  // A packing workgroup moves TRTRI_PACK_EACH blocks, one after the other (a few microseconds
  // each): only one workgroup fits a CU, and with one per block a call with 1024-row panels
  // would have more workgroups than the device has CUs, the last inversions waiting for a CU.
  const int ndiag = (na + NB - 1) / NB, npack = (int)gridDim.x - ndiag;
  const int pairs = panel_pairs(panel_blocks);
  const int npair_all = ((na + panel_blocks * NB - 1) / (panel_blocks * NB)) * pairs;
  // Pack role: block (hi, lo) of a panel, hi > lo, on the side of the diagonal M has.
  auto pack_block = [&](int idx) {
    const int panel = idx / pairs, pair = idx % pairs;
    int hi = 1;
    while ((hi + 1) * hi / 2 <= pair) ++hi;
    const int lo = pair - hi * (hi - 1) / 2;
    const bool m_lower = (lower != 0) != (mtrans != 0);
    const int br = panel * panel_blocks + (m_lower ? hi : lo);  // block row / column within M
    const int bc = panel * panel_blocks + (m_lower ? lo : hi);
    T* dst = packed + ((long)panel * pairs + pair) * NB * NB;
    const int tt = threadIdx.x;
    // 32 loads are in flight per lane: a loop that waits for each element would make this
    // role, which moves 128 KiB a block, last longer than an inversion.
    constexpr int INFL = 32;
    if (!mtrans) {
      // dst(r, c) = A(br*NB + r, bc*NB + c): rows along the lanes on both sides.
      const int r = tt & (NB - 1);
      const long gr = (long)br * NB + r;
      for (int c0 = tt >> 7; c0 < NB; c0 += 2 * INFL) {
        T v[INFL];
#pragma unroll
        for (int u = 0; u < INFL; ++u) {
          const long gc = (long)bc * NB + c0 + 2 * u;
          v[u] = (gr < na && gc < na) ? A[gr + gc * lda] : T(0);
        }
#pragma unroll
        for (int u = 0; u < INFL; ++u) dst[block_offset<T>(r, c0 + 2 * u, frag)] = v[u];
      }
    } else {
      // dst(r, c) = A(bc*NB + c, br*NB + r): through LDS, so that both sides run along lanes.
      const int c = tt & (NB - 1);
      const long gc = (long)bc * NB + c;
      for (int r0 = tt >> 7; r0 < NB; r0 += 2 * INFL) {
        T v[INFL];
#pragma unroll
        for (int u = 0; u < INFL; ++u) {
          const long gr = (long)br * NB + r0 + 2 * u;
          v[u] = (gr < na && gc < na) ? A[gc + gr * lda] : T(0);
        }
#pragma unroll
        for (int u = 0; u < INFL; ++u) L[c + (r0 + 2 * u) * LD] = v[u];
      }
      __syncthreads();
      const int r = tt & (NB - 1);
      for (int cc = tt >> 7; cc < NB; cc += 2) dst[block_offset<T>(r, cc, frag)] = L[cc + r * LD];
      __syncthreads();  // L is free for the next block
    }
  };
  if ((int)blockIdx.x < npack) {
    const int first = (int)blockIdx.x * TRTRI_PACK_EACH;
    for (int idx = first; idx < first + TRTRI_PACK_EACH && idx < npair_all; ++idx) pack_block(idx);
    return;
  }
  const int blk = (int)blockIdx.x - npack;
  const int b0 = blk * NB;
  const int nb = (na - b0 < NB) ? na - b0 : NB;
  const int t = threadIdx.x;
  const int i = t & (NB - 1), half = t >> 7;  // two lanes per row
  const T* Ab = A + b0 + (long)b0 * lda;

  // The diagonal element of this lane's row, requested ahead of the triangle so that it does
  // not cost a second trip to memory behind the first barrier.
  T d = T(1);
  if (half == 0 && i < nb && !unit) d = Ab[i + (long)i * lda];

  // Load the strict triangle (coalesced along the stored columns), zero the rest; rows and
  // columns past the end of A become identity.  32 columns are in flight per lane.
  constexpr int INFL = 32;
  for (int c0 = half; c0 < NB; c0 += 2 * INFL) {
    T v[INFL];
#pragma unroll
    for (int u = 0; u < INFL; ++u) {
      const int c = c0 + 2 * u;
      const bool wanted = i < nb && c < nb && (lower ? c < i : i < c);
      v[u] = wanted ? Ab[i + (long)c * lda] : T(0);
    }
#pragma unroll
    for (int u = 0; u < INFL; ++u) {
      const int c = c0 + 2 * u;
      if (lower) L[i + c * LD] = v[u];
      else L[c + i * LD] = v[u];
    }
  }
  __syncthreads();
  if (half == 0) {
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
  const bool out_lower = (lower != 0) != (mtrans != 0);  // triangle of inv(M_ii)
  for (int k = half; k < NB; k += 2) {
    // lower: O(i,k) = L(i,k) for k <= i; upper: O(i,k) = L(k,i) for i <= k; zero elsewhere.
    T v = T(0);
    if (out_lower) {
      if (k <= i) v = L[i + k * LD];
    } else {
      if (i <= k) v = L[k + i * LD];
    }
    O[block_offset<T>(i, k, frag)] = v;
  }
}

// ---- panel solve -----------------------------------------------------------------------

constexpr int PANEL_THREADS = 256;   // 4 waves: wave w owns rows 32w .. 32w+31 of every block
constexpr int PANEL_W = 16;          // right-hand sides per workgroup

template <class T>
struct PanelArgs {
  const T* inv;     // inverses of the panel's diagonal blocks in M's orientation, NB*NB each
  const T* packed;  // the panel's off-diagonal blocks of M (trtri_kernel's pack role)
  int rows;         // rows of the panel (<= the kernel's panel height)
  T* B;             // element (panel row 0, right-hand side 0)
  long sp, sw;      // strides of B along the panel rows / along the right-hand sides
  int nrhs;         // number of right-hand sides
  int forward;      // 1: M is lower triangular (blocks 0, 1, ...); 0: upper (last block first)
};

// Element-wise LDS stride of one right-hand side: the panel's rows plus a pad that makes the
// stride 8 banks (mod 64), the lane stride under which 16-byte reads by 16 lanes are conflict
// free.
template <class T, int PR> struct PanelLd { static constexpr int LD = PR + 32 / (int)sizeof(T); };
// Workgroups of a panel kernel that fit a CU (160 KiB of LDS).
template <class T, int PR> struct PanelFit {
  static constexpr int PER_CU =
      (160 * 1024) / (PANEL_W * PanelLd<T, PR>::LD * (int)sizeof(T)) >= 2 ? 2 : 1;
};

// One workgroup solves the panel for PANEL_W right-hand sides, which it keeps in LDS.  A wave
// owns 32 rows of every 128-row block as two MFMA blocks with interleaved rows (rows 2l and
// 2l+1 of the 32 belong to lane l of block 0 and block 1).  Where two workgroups fit a CU, one's
// barriers and LDS phases overlap the other's MFMAs.  PR: the panel height in rows.
template <class T, int PR>
__global__ __launch_bounds__(PANEL_THREADS, (PanelFit<T, PR>::PER_CU)) void trsm_panel_kernel(
    PanelArgs<T> p) {
  constexpr int PANEL = PR;
  constexpr int E = Elem<T>::E, LD = PanelLd<T, PR>::LD, W = PANEL_W, STEPS = NB / 4, NGRP = STEPS / E;
  typedef typename Elem<T>::acc_t acc_t;
  typedef typename VecOf<T, E>::type vec_t;
  typedef typename VecOf<T, 2>::type pair_t;
  extern __shared__ __align__(16) unsigned char panel_raw[];
  T* S = reinterpret_cast<T*>(panel_raw);  // S[w * LD + r]: right-hand side w, panel row r

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int r16 = lane & 15, kq = lane >> 4;
  const int w0 = blockIdx.x * W;
  const int nblk = (p.rows + NB - 1) / NB;

  // Slab in: rows past the panel's end and right-hand sides past nrhs are zero.  Eight
  // loads are in flight per lane (addresses clamped, values selected afterwards).
  if (p.sp == 1) {
#pragma unroll 1
    for (int rb = 0; rb < PANEL; rb += PANEL_THREADS) {
      const int r = rb + t;
      const bool row_ok = r < p.rows;
      const long row = row_ok ? r : 0;
#pragma unroll 1
      for (int wb = 0; wb < W; wb += 8) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int w = w0 + wb + u;
          v[u] = p.B[row + (long)(w < p.nrhs ? w : 0) * p.sw];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          S[(wb + u) * LD + r] = (row_ok && w0 + wb + u < p.nrhs) ? v[u] : T(0);
      }
    }
  } else {
    const int w = t % W;
    const bool w_ok = w0 + w < p.nrhs;
    const long wc = w_ok ? w0 + w : 0;
    constexpr int RSTEP = PANEL_THREADS / W;
#pragma unroll 1
    for (int rb = t / W; rb < PANEL; rb += 8 * RSTEP) {
      T v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int r = rb + u * RSTEP;
        v[u] = p.B[(long)(r < p.rows ? r : 0) * p.sp + wc * p.sw];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int r = rb + u * RSTEP;
        S[w * LD + r] = (w_ok && r < p.rows) ? v[u] : T(0);
      }
    }
  }

  // k index of MFMA step s for this lane group: steps in groups of E take neighbouring k.
  auto step_k = [&](int s) { return 4 * E * (s / E) + E * kq + s % E; };

  // The A-slot values of one block product Out = Aop * In: Aop(row + i, k), i = 0, 1 (the
  // lane's two rows, neighbours in memory), of a 128 x 128 column-major block in scratch: a
  // diagonal-block inverse (leaf) or an off-diagonal block of M (update).
  auto block_of = [&](int idx) { return p.forward ? idx : nblk - 1 - idx; };
  auto source_of = [&](int step, int u) -> const T* {
    const int out = block_of(u), in = block_of(step);
    const T* blk;
    if (u == step) {
      blk = p.inv + (long)out * NB * NB;
    } else {
      const int hi = out > in ? out : in, lo = out > in ? in : out;
      blk = p.packed + (long)(hi * (hi - 1) / 2 + lo) * NB * NB;
    }
    return blk + 32 * wave + 2 * r16;
  };

  // The A-slot values of step group g from block column base `a` into af[g*E .. g*E+E-1][0..1].
  auto fetch_group = [&](const T* a, int g, T (&af)[STEPS][2]) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const pair_t v = *reinterpret_cast<const pair_t*>(a + step_k(g * E + e) * NB);
      af[g * E + e][0] = v[0];
      af[g * E + e][1] = v[1];
    }
  };

  // One block product, acc = Aop * S(rows of block `in`) with the A-slot values in af.  As
  // soon as the MFMAs of a step group have read their values, the same registers are refilled
  // with the NEXT product's values: the global loads trail the MFMAs a group at a time and
  // have a whole product's time to arrive.
  auto product = [&](int in, T (&af)[STEPS][2], acc_t (&acc)[2], const T* nx) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][r] = T(0);
    const T* sin = S + r16 * LD + in * NB + E * kq;
    vec_t bf[2];
    bf[0] = *reinterpret_cast<const vec_t*>(sin);
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      if (g + 1 < NGRP) bf[(g + 1) & 1] = *reinterpret_cast<const vec_t*>(sin + 4 * E * (g + 1));
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int i = 0; i < 2; ++i)
          acc[i] = Elem<T>::mfma(af[g * E + e][i], bf[g & 1][e], acc[i]);
      fetch_group(nx, g, af);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // The wave's elements of block `out`: lane holds rows 2*rho and 2*rho+1 (rho = acc_row(r, lane))
  // of its 32, right-hand side lane % 16, as a pair.
  auto slab_pair = [&](int out, int r) -> pair_t* {
    return reinterpret_cast<pair_t*>(S + r16 * LD + out * NB + 32 * wave +
                                     2 * Elem<T>::acc_row(r, lane));
  };

  // The block products of the panel in order: for each block i (first to last, or last to
  // first for an upper triangular M) the leaf X_i = inv(M_ii) B_i, then the updates
  // B_o -= M(o, i) X_i of the blocks still to be solved.  (step, u): u == step is the leaf of
  // step, u > step the update of the u-th block.  The last product refills with its own
  // values (a fetch without a branch keeps each product free of control flow).
  auto advance = [&](int& step, int& u) {
    if (++u >= nblk) u = ++step;
  };
  T af[STEPS][2];
  int step = 0, u = 0;
  if (nblk > 0) {
    const T* a0 = source_of(0, 0);
#pragma unroll
    for (int g = 0; g < NGRP; ++g) fetch_group(a0, g, af);
  }
  while (step < nblk) {
    int ns = step, nu = u;
    advance(ns, nu);
    const T* nx = ns < nblk ? source_of(ns, nu) : source_of(step, u);
    acc_t acc[2];
    const int i = block_of(step), o = block_of(u);
    const bool leaf = u == step;
    if (leaf) __syncthreads();  // the slab (first step) or the updates of block i are in
    product(i, af, acc, nx);
    if (leaf) {
      __syncthreads();  // all waves have read B_i: it may be overwritten
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pair_t v;
        v[0] = acc[0][r];
        v[1] = acc[1][r];
        *slab_pair(i, r) = v;
      }
      __syncthreads();
    } else {  // each lane owns its elements of B_o
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pair_t* q = slab_pair(o, r);
        pair_t v = *q;
        v[0] -= acc[0][r];
        v[1] -= acc[1][r];
        *q = v;
      }
    }
    step = ns;
    u = nu;
  }
  __syncthreads();

  // Slab out.
  if (p.sp == 1) {
    for (int r = t; r < PANEL; r += PANEL_THREADS)
      for (int w = 0; w < W; ++w)
        if (r < p.rows && w0 + w < p.nrhs) p.B[(long)r + (long)(w0 + w) * p.sw] = S[w * LD + r];
  } else {
    const int w = t % W;
    for (int r = t / W; r < PANEL; r += PANEL_THREADS / W)
      if (r < p.rows && w0 + w < p.nrhs) p.B[(long)r * p.sp + (long)(w0 + w) * p.sw] = S[w * LD + r];
  }
}

template <class T, int PR>
static rtat_status_t launch_panel(rtat_native_handle* h, const PanelArgs<T>& a) {
  const size_t lds_bytes = (size_t)PANEL_W * PanelLd<T, PR>::LD * sizeof(T);
  auto kern = trsm_panel_kernel<T, PR>;
  // The attribute is per device; a handle is bound to the device it was created on.
  static PerDeviceOnce configured;
  if (!configured(h->device, [&] {
        if (lds_bytes <= 65536) return true;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) == hipSuccess)
          return true;
        (void)hipGetLastError();
        return false;
      }))
    return RTAT_STATUS_NOT_SUPPORTED;
  const unsigned grid = (unsigned)((a.nrhs + PANEL_W - 1) / PANEL_W);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(PANEL_THREADS), lds_bytes, h->stream, a);
  return launch_status();
}

// ---- wide panel solve --------------------------------------------------------------------

constexpr int WIDE_THREADS = 512;  // 8 waves: wave v owns rows 16v .. 16v+15 of every block
constexpr int WIDE_W = 32;         // right-hand sides per workgroup: two MFMA column tiles
template <class T> struct WideLd { static constexpr int LD = NB + 32 / (int)sizeof(T); };

// The panel solve for many right-hand sides (512-row panels, more than one 16-wide slab per
// CU).  One workgroup per CU solves the panel for 32 right-hand sides.  A wave owns 16 rows of
// every 128-row block and both column tiles, so every value of M it loads feeds two MFMAs; its
// part of the panel stays in registers from the load to the store (res[block][column tile]),
// and only the block in flight crosses LDS: B_i on its way into the product with inv(M_ii)
// (buffer P), -X_i on its way into the updates (buffer Q), which accumulate straight into
// res.  The loads of the later blocks and the stores of the solved ones trail the products;
// the two waves of a SIMD cover each other's LDS and issue latencies.
//   NBLK  blocks of the panel (ceil(rows / 128)): the whole substitution is straight-line code.
//   SWAP  the MFMAs compute the transposed products, which puts the lanes along the panel
//         rows and the registers along the right-hand sides.  Either way the lanes run along
//         the dimension that is contiguous in B: SWAP for a left-hand solve (rows), not for
//         a right-hand one (right-hand sides).
template <class T, int NBLK, bool SWAP>
__global__ __launch_bounds__(WIDE_THREADS, 1) void trsm_panel_wide_kernel(PanelArgs<T> p) {
  constexpr int E = Elem<T>::E, LD = WideLd<T>::LD, W = WIDE_W, STEPS = NB / 4, NGRP = STEPS / E;
  typedef typename Elem<T>::acc_t acc_t;
  typedef typename VecOf<T, E>::type vec_t;
  extern __shared__ __align__(16) unsigned char panel_raw[];
  T* P = reinterpret_cast<T*>(panel_raw);  // P[w * LD + r]: right-hand side w, block row r
  T* Q = P + W * LD;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int r16 = lane & 15, kq = lane >> 4;
  const int w0 = blockIdx.x * W;
  // The lane feeds row 16 wave + r16 of M to every MFMA.  Without SWAP its register r holds
  // block row 16 wave + acc_row(r, lane), right-hand side 16c + r16.  Under SWAP the registers
  // run along the right-hand sides: the MFMA's index rho of that dimension is fed right-hand
  // side pi(rho) of the tile's sixteen, pi chosen so that the lane's four results are the
  // neighbours 4kq .. 4kq+3 (double: register r holds rho = 4r + kq; float: rho = 4kq + r), and
  // register r holds block row 16 wave + r16, right-hand side 16c + 4kq + r.
  const int pi16 = sizeof(T) == 8 ? 4 * (r16 & 3) + (r16 >> 2) : r16;
  const int bcol = SWAP ? pi16 : r16;  // right-hand side (of a tile) the lane feeds
  auto row_of = [&](int r) { return 16 * wave + (SWAP ? r16 : Elem<T>::acc_row(r, lane)); };
  auto col_of = [&](int r) { return SWAP ? 4 * kq + r : r16; };
  // The lane's part of an address inside a block of M in fragment order (frag_offset); the
  // rest is the same for all lanes, so a load is a scalar base plus this offset.
  const unsigned lane_off = (unsigned)((wave * NGRP * 64 + lane) * E);

  auto block_of = [&](int idx) { return p.forward ? idx : NBLK - 1 - idx; };
  // Block of M behind the product (step, u): u == step the inverse of diagonal block step,
  // u > step the off-diagonal block that updates the u-th block with the step-th solution.
  auto source_of = [&](int step, int u) -> const T* {
    const int out = block_of(u), in = block_of(step);
    if (u == step) return p.inv + (long)out * NB * NB;
    const int hi = out > in ? out : in, lo = out > in ? in : out;
    return p.packed + (long)(hi * (hi - 1) / 2 + lo) * NB * NB;
  };
  // MFMA step s = g * E + e of a product takes k = 4E g + E kq + e: a lane's E values of a
  // group are neighbours in LDS and in the block of M, one 16-byte access each.
  auto fetch_group = [&](const T* blk, int g, T (&af)[STEPS]) {
    const vec_t v = *reinterpret_cast<const vec_t*>(blk + g * 64 * E + lane_off);
#pragma unroll
    for (int e = 0; e < E; ++e) af[g * E + e] = v[e];
  };
  // acc[c] += Mblock * buf for both column tiles; as soon as the MFMAs of a group have read
  // their values of M, the same registers are refilled with the next product's.
  auto product = [&](const T* buf, T (&af)[STEPS], acc_t (&acc)[2], const T* nx) {
    const T* sin = buf + bcol * LD + E * kq;
    vec_t bf[2][2];
#pragma unroll
    for (int c = 0; c < 2; ++c) bf[0][c] = *reinterpret_cast<const vec_t*>(sin + 16 * c * LD);
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      if (g + 1 < NGRP) {
#pragma unroll
        for (int c = 0; c < 2; ++c)
          bf[(g + 1) & 1][c] =
              *reinterpret_cast<const vec_t*>(sin + 16 * c * LD + 4 * E * (g + 1));
      }
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int c = 0; c < 2; ++c)
          acc[c] = SWAP ? Elem<T>::mfma(bf[g & 1][c][e], af[g * E + e], acc[c])
                        : Elem<T>::mfma(af[g * E + e], bf[g & 1][c][e], acc[c]);
      fetch_group(nx, g, af);
      // Issue order inside the group: the LDS reads of the next group first, then the MFMAs
      // with the refill behind the first of them.
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * E - 1, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Where the lane's element (block idx, column tile c, register r) lives in B, and whether
  // it exists (rows past the panel's end and right-hand sides past nrhs do not).
  auto place = [&](int idx, int c, int r, long& off) -> bool {
    const int row = block_of(idx) * NB + row_of(r);
    const int w = w0 + 16 * c + col_of(r);
    const bool ok = row < p.rows && w < p.nrhs;
    off = ok ? (long)row * p.sp + (long)w * p.sw : 0;
    return ok;
  };
  // The lane's values of a block, times sign, to an LDS buffer.
  auto park = [&](T* buf, const acc_t (&v)[2], T sign) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) buf[(16 * c + col_of(r)) * LD + row_of(r)] = sign * v[c][r];
  };

  acc_t res[NBLK][2];
  T af[STEPS];
  auto load_block = [&](int idx) {  // addresses clamped; mask_block zeroes what does not exist
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        long off;
        (void)place(idx, c, r, off);
        res[idx][c][r] = p.B[off];
      }
  };
  auto mask_block = [&](int idx) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        long off;
        if (!place(idx, c, r, off)) res[idx][c][r] = T(0);
      }
  };

  // Loads return in order: the first block and the first inverse are asked for first, and
  // the first product starts while the other blocks are still on their way.
  load_block(0);
  {
    const T* a0 = source_of(0, 0);
#pragma unroll
    for (int g = 0; g < NGRP; ++g) fetch_group(a0, g, af);
  }
  constexpr int EARLY = NBLK < 4 ? NBLK : 4;  // blocks asked for before the first product
#pragma unroll
  for (int idx = 1; idx < EARLY; ++idx) load_block(idx);
  __builtin_amdgcn_sched_barrier(0);
  mask_block(0);

#pragma unroll
  for (int i = 0; i < NBLK; ++i) {
    // Leaf: X_i = inv(M_ii) B_i.  P was last read by the previous leaf, which every wave has
    // left behind at the barrier that followed it.
    park(P, res[i], T(1));
    __syncthreads();
    {
      const T* nx = i + 1 < NBLK ? source_of(i, i + 1) : source_of(i, i);
      acc_t acc[2];
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[c][r] = T(0);
      product(P, af, acc, nx);
      res[i][0] = acc[0];
      res[i][1] = acc[1];
    }
    if (i + 1 < NBLK) {
      // Q was last read by the updates with X_(i-1), which every wave finished before the
      // barrier in front of this leaf.
      park(Q, res[i], T(-1));
      __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        long off;
        if (place(i, c, r, off)) p.B[off] = res[i][c][r];
      }
    if (i == 0) {
      // The rest of a tall panel is asked for now (a wave can have 63 loads in flight): block
      // u is first used u products from here.
#pragma unroll
      for (int idx = EARLY; idx < NBLK; ++idx) load_block(idx);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Updates: B_u -= M(u, i) X_i, accumulated in place.
#pragma unroll
    for (int u = i + 1; u < NBLK; ++u) {
      const T* nx = u + 1 < NBLK ? source_of(i, u + 1) : source_of(i + 1, i + 1);
      if (i == 0) mask_block(u);
      product(Q, af, res[u], nx);
    }
  }
}

template <class T, int NBLK, bool SWAP>
static rtat_status_t launch_panel_wide_as(rtat_native_handle* h, const PanelArgs<T>& a) {
  const size_t lds_bytes = (size_t)2 * WIDE_W * WideLd<T>::LD * sizeof(T);
  auto kern = trsm_panel_wide_kernel<T, NBLK, SWAP>;
  // The attribute is per device; a handle is bound to the device it was created on.
  static PerDeviceOnce configured;
  if (!configured(h->device, [&] {
        if (lds_bytes <= 65536) return true;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) == hipSuccess)
          return true;
        (void)hipGetLastError();
        return false;
      }))
    return RTAT_STATUS_NOT_SUPPORTED;
  const unsigned grid = (unsigned)((a.nrhs + WIDE_W - 1) / WIDE_W);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(WIDE_THREADS), lds_bytes, h->stream, a);
  return launch_status();
}

template <class T, int NBLK>
static rtat_status_t launch_panel_wide_n(rtat_native_handle* h, const PanelArgs<T>& a) {
  return a.sp == 1 ? launch_panel_wide_as<T, NBLK, true>(h, a)
                   : launch_panel_wide_as<T, NBLK, false>(h, a);
}

template <class T>
static rtat_status_t launch_panel_wide(rtat_native_handle* h, const PanelArgs<T>& a) {
  static_assert(PANEL_TALL == 8 * NB, "one instantiation per block count of a panel");
  switch ((a.rows + NB - 1) / NB) {
    case 1: return launch_panel_wide_n<T, 1>(h, a);
    case 2: return launch_panel_wide_n<T, 2>(h, a);
    case 3: return launch_panel_wide_n<T, 3>(h, a);
    case 4: return launch_panel_wide_n<T, 4>(h, a);
    case 5: return launch_panel_wide_n<T, 5>(h, a);
    case 6: return launch_panel_wide_n<T, 6>(h, a);
    case 7: return launch_panel_wide_n<T, 7>(h, a);
    case 8: return launch_panel_wide_n<T, 8>(h, a);
  }
  return RTAT_STATUS_INVALID_VALUE;
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
  const T* packed;
  int variant;
  int panel;  // panel height of this call: PANEL_SHORT or PANEL_TALL
  bool wide;  // short panels by trsm_panel_wide_kernel
  rtat_status_t st;
};

static inline int split_point(int lo, int hi, int panel) {
  const int panels = (hi - lo + panel - 1) / panel;
  return lo + panel * ((panels + 1) / 2);
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
  if (len <= c.panel) {
    PanelArgs<T> a;
    a.inv = c.inv + (long)(lo / NB) * NB * NB;
    a.packed = c.packed + (long)(lo / c.panel) * panel_pairs(c.panel / NB) * NB * NB;
    a.rows = len;
    const bool eff_lower = c.lower != c.trans;
    if (c.left) {
      a.B = c.B + lo;
      a.sp = 1;
      a.sw = c.ldb;
      a.nrhs = c.n;
      a.forward = eff_lower ? 1 : 0;
    } else {
      a.B = c.B + (long)lo * c.ldb;
      a.sp = c.ldb;
      a.sw = 1;
      a.nrhs = c.m;
      a.forward = eff_lower ? 0 : 1;
    }
    c.st = c.wide                  ? launch_panel_wide<T>(c.h, a)
           : c.panel == PANEL_TALL ? launch_panel<T, PANEL_TALL>(c.h, a)
                                   : launch_panel<T, PANEL_SHORT>(c.h, a);
    return;
  }
  const int mid = split_point(lo, hi, c.panel);
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

// What a caller that lends the scratch has to provide: enough for either panel height.
size_t trsm_workspace_bytes(int na) {
  if (na <= 0) return 0;
  return trsm_scratch_elems(na, PANEL_TALL, nullptr) * sizeof(double) + 16;  // float: half of it
}

// Which kernel solves the panels.  The wide kernel needs half as many workgroups as the 16-wide
// one for the same right-hand sides and runs one per CU, whatever the panel height: it is
// taken where the 16-wide one would put more than one workgroup on a CU.
static bool wide_panels(const rtat_native_handle* h, int nrhs) {
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  return (nrhs + PANEL_W - 1) / PANEL_W > cus;
}

// Panel height of a call.  The tall panel saves a level of GEMM updates.  The wide kernel
// runs it as fast per block product as the short one, so it always takes it (measured on
// MI355X, 8192 right-hand sides: two 512-row panels and the 512-deep update between them 48 +
// 68 + 48 us, one 1024-row panel 152 us; DTRSM n = 8192 7.83 -> 7.77 ms, STRSM 4.16 -> 3.9).
// The 16-wide kernel keeps its slab in LDS and runs a tall panel one workgroup per CU in double
// precision: it pays when the right-hand sides give at most one workgroup per CU anyway (in
// single precision two tall workgroups fit a CU, and any larger number will do).  With fewer
// workgroups than half the CUs the panel kernel leaves most of the machine idle, and the
// update it would absorb is better off as a GEMM over all CUs.  Measured: DTRSM n = 4096
// 1.21 -> 1.16 ms, STRSM n = 4096 0.70 -> 0.68 ms.
template <class T>
static int pick_panel(const rtat_native_handle* h, int nrhs) {
  if (wide_panels(h, nrhs)) return PANEL_TALL;
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  const long groups = (nrhs + PANEL_W - 1) / PANEL_W;
  if (2 * groups <= cus) return PANEL_SHORT;
  if (PanelFit<T, PANEL_TALL>::PER_CU >= 2) return PANEL_TALL;
  return groups <= cus ? PANEL_TALL : PANEL_SHORT;
}

template <class T>
rtat_status_t launch_trsm(rtat_native_handle* h, bool left, bool lower, bool trans, bool unit,
                          int m, int n, T alpha, const T* A, int lda, T* B, int ldb,
                          int variant) {
  if (m < 0 || n < 0 || ldb < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  KernelOptions opt;
  if (!decode_options(variant, opt)) return RTAT_STATUS_INVALID_VALUE;
  // The trailing updates get the tile shape and the tail mode; the panel height is ours.
  variant = RTAT_KERNEL_OPTIONS(opt.tile, opt.tail, RTAT_PANEL_AUTO);
  const int na = left ? m : n;
  if (lda < (na > 1 ? na : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (B == nullptr) return RTAT_STATUS_INVALID_VALUE;
  if (alpha == T(0))
    return launch_geam<T>(h, false, false, m, n, T(0), nullptr, 0, T(0), nullptr, 0, B, ldb);
  if (A == nullptr) return RTAT_STATUS_INVALID_VALUE;

  const int panel = opt.panel == RTAT_PANEL_512    ? PANEL_SHORT
                    : opt.panel == RTAT_PANEL_1024 ? PANEL_TALL
                                                   : pick_panel<T>(h, left ? n : m);
  h->last.trsm_panel_rows = panel;
  const bool wide = wide_panels(h, left ? n : m);
  h->last.trsm_panel_width = wide ? WIDE_W : PANEL_W;
  size_t packed_offset = 0;
  const size_t need = trsm_scratch_elems(na, panel, &packed_offset) * sizeof(T) + 16;
  void* raw = acquire_workspace(h, need);
  if (raw == nullptr) return RTAT_STATUS_ALLOC_FAILED;
  // The panel kernel reads scratch with 16-byte accesses: align a lent buffer up.
  T* inv = reinterpret_cast<T*>((reinterpret_cast<uintptr_t>(raw) + 15) & ~(uintptr_t)15);
  T* packed = inv + packed_offset;

  static PerDeviceOnce configured;
  const size_t lds_bytes = TRTRI_LDS_ELEMS * sizeof(T);
  if (!configured(h->device, [&] {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(trtri_kernel<T>),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) == hipSuccess)
          return true;
        (void)hipGetLastError();
        return false;
      }))
    return RTAT_STATUS_NOT_SUPPORTED;
  // M = op'(A) is the system matrix of the left-hand form: a right-hand solve X op(A) = B is
  // op(A)^T X^T = B^T.
  const bool mtrans = left ? trans : !trans;
  const int nblk = (na + NB - 1) / NB, npanel = (na + panel - 1) / panel;
  const int npack = (npanel * panel_pairs(panel / NB) + TRTRI_PACK_EACH - 1) / TRTRI_PACK_EACH;
  hipLaunchKernelGGL(trtri_kernel<T>, dim3(nblk + npack),
                     dim3(TRTRI_THREADS), lds_bytes, h->stream, A, (long)lda, na, lower ? 1 : 0,
                     unit ? 1 : 0, mtrans ? 1 : 0, inv, packed, panel / NB, wide ? 1 : 0);
  rtat_status_t st = launch_status();
  if (st != RTAT_STATUS_SUCCESS) return st;

  if (alpha != T(1)) {
    st = launch_geam<T>(h, false, false, m, n, alpha, B, ldb, T(0), nullptr, 0, B, ldb);
    if (st != RTAT_STATUS_SUCCESS) return st;
  }
  TrsmCtx<T> c{h,   left, lower, trans,  m,       n,     A,
               lda, B,    ldb,   inv,    packed,  variant, panel, wide,
               RTAT_STATUS_SUCCESS};
  solve_range(c, 0, na);
  return c.st;
}

template rtat_status_t launch_trsm<double>(rtat_native_handle*, bool, bool, bool, bool, int, int,
                                           double, const double*, int, double*, int, int);
template rtat_status_t launch_trsm<float>(rtat_native_handle*, bool, bool, bool, bool, int, int,
                                          float, const float*, int, float*, int, int);

}  // namespace rtat_native
