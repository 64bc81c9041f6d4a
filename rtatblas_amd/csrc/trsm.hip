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
//      a slab of 16 or 32 of them, holds the slab's panel rows in registers and runs the whole
//      blocked substitution on it (X_i = inv(M_ii) B_i, B_j -= M_ji X_i for the blocks of the
//      panel) with MFMAs; only the block in flight crosses LDS.  The blocks of M it needs (the
//      inverses and the off-diagonal blocks inside each panel) are laid out once per call, by
//      the launch that inverts the diagonal blocks, in scratch, in the order the panel
//      kernel's lanes consume them; all workgroups read them, so they live in L2.
//   All sixteen side / uplo / trans / diag combinations run natively and alike: a right-hand
//   solve is the left-hand solve of the transposed system (the slab is held transposed,
//   M = op(A)^T), trans flips the effective triangle, inv(op(T)) = op(inv(T)).
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
// Both kinds of block are written in the order trsm_panel_kernel's lanes consume them
// (frag_offset).
template <class T>
__global__ __launch_bounds__(TRTRI_THREADS) void trtri_kernel(const T* A, long lda, int na, int lower,
                                                             int unit, int mtrans, T* out,
                                                             T* packed, int panel_blocks) {
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
    // All of a lane's 64 loads are in flight at once: a loop that waits for each element would
    // make this role, which moves 128 KiB a block, last longer than an inversion.  A lane owns
    // row r of every second group of E columns (E = elements per 16 bytes), which the
    // fragment order keeps together: one 16-byte store per group.
    constexpr int E = Elem<T>::E, GROUPS = NB / E / 2;
    typedef typename VecOf<T, E>::type vec_t;
    const int r = tt & (NB - 1), h = tt >> 7;
    T v[GROUPS][E];
    if (!mtrans) {
      // dst(r, c) = A(br*NB + r, bc*NB + c): rows along the lanes on both sides.
      const long gr = (long)br * NB + r;
#pragma unroll
      for (int u = 0; u < GROUPS; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const long gc = (long)bc * NB + E * (h + 2 * u) + e;
          v[u][e] = (gr < na && gc < na) ? A[gr + gc * lda] : T(0);
        }
    } else {
      // dst(r, c) = A(bc*NB + c, br*NB + r): through LDS, so that both sides run along lanes.
      const long gc = (long)bc * NB + r;  // this lane's column of M = row of A
#pragma unroll
      for (int u = 0; u < GROUPS; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const long gr = (long)br * NB + E * (h + 2 * u) + e;
          v[u][e] = (gr < na && gc < na) ? A[gc + gr * lda] : T(0);
        }
#pragma unroll
      for (int u = 0; u < GROUPS; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) L[r + (E * (h + 2 * u) + e) * LD] = v[u][e];
      __syncthreads();
#pragma unroll
      for (int u = 0; u < GROUPS; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) v[u][e] = L[(E * (h + 2 * u) + e) + r * LD];
      __syncthreads();  // L is free for the next block
    }
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) {
      vec_t x;
#pragma unroll
      for (int e = 0; e < E; ++e) x[e] = v[u][e];
      *reinterpret_cast<vec_t*>(dst + frag_offset<T>(r, E * (h + 2 * u))) = x;
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
  // columns past the end of A become identity.  All 64 columns of a lane are in flight at once.
  constexpr int INFL = NB / 2;
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
  constexpr int E = Elem<T>::E;
  typedef typename VecOf<T, E>::type vec_t;
#pragma unroll 8
  for (int kp = half; kp < NB / E; kp += 2) {  // E neighbouring k: one 16-byte store
    vec_t x;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      // lower: O(i,k) = L(i,k) for k <= i; upper: O(i,k) = L(k,i) for i <= k; zero elsewhere.
      const int k = kp * E + e;
      T v = T(0);
      if (out_lower) {
        if (k <= i) v = L[i + k * LD];
      } else {
        if (i <= k) v = L[k + i * LD];
      }
      x[e] = v;
    }
    *reinterpret_cast<vec_t*>(O + frag_offset<T>(i, kp * E)) = x;
  }
}

// ---- panel solve -----------------------------------------------------------------------

constexpr int PANEL_THREADS = 512;  // 8 waves: wave v owns rows 16v .. 16v+15 of every block
constexpr int PANEL_W = 16;         // right-hand sides per MFMA column tile

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

// Element-wise LDS stride of one right-hand side: a block's rows plus a pad that makes the
// stride 8 banks (mod 64).
template <class T> struct PanelLd { static constexpr int LD = NB + 32 / (int)sizeof(T); };

// The panel solve.  Right-hand sides are independent, so each workgroup (one per CU) takes a
// slab of 16 NC of them and runs the whole blocked substitution on it.  A wave owns 16 rows of
// every 128-row block and all NC column tiles, so every value of M it loads feeds NC MFMAs;
// its part of the slab stays in registers from the load to the store (res[block][column
// tile]), and only the block in flight crosses LDS: B_i on its way into the product with
// inv(M_ii) (buffer P), -X_i on its way into the updates (buffer Q), which accumulate straight
// into res.  The loads of the later blocks and the stores of the solved ones trail the
// products; the two waves of a SIMD cover each other's LDS and issue latencies.
//   NBLK  blocks of the panel (ceil(rows / 128)): the whole substitution is straight-line code.
//   SWAP  the MFMAs compute the transposed products, which puts the lanes along the panel
//         rows and the registers along the right-hand sides.  Either way the lanes run along
//         the dimension that is contiguous in B: SWAP for a left-hand solve (rows), not for
//         a right-hand one (right-hand sides).
//   NC    column tiles per workgroup: 2 when 16 right-hand sides per workgroup would give more
//         workgroups than CUs (half the traffic from L2 per flop), else 1 (more workgroups).
template <class T, int NBLK, bool SWAP, int NC>
__global__ __launch_bounds__(PANEL_THREADS, 1) void trsm_panel_kernel(PanelArgs<T> p) {
  constexpr int E = Elem<T>::E, LD = PanelLd<T>::LD, W = PANEL_W * NC, STEPS = NB / 4, NGRP = STEPS / E;
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
  // acc[c] += Mblock * buf for every column tile; as soon as the MFMAs of a group have read
  // their values of M, the same registers are refilled with the next product's.
  auto product = [&](const T* buf, T (&af)[STEPS], acc_t (&acc)[NC], const T* nx) {
    const T* sin = buf + bcol * LD + E * kq;
    vec_t bf[2][NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) bf[0][c] = *reinterpret_cast<const vec_t*>(sin + 16 * c * LD);
#pragma unroll
    for (int g = 0; g < NGRP; ++g) {
      if (g + 1 < NGRP) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
          bf[(g + 1) & 1][c] =
              *reinterpret_cast<const vec_t*>(sin + 16 * c * LD + 4 * E * (g + 1));
      }
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int c = 0; c < NC; ++c)
          acc[c] = SWAP ? Elem<T>::mfma(bf[g & 1][c][e], af[g * E + e], acc[c])
                        : Elem<T>::mfma(af[g * E + e], bf[g & 1][c][e], acc[c]);
      fetch_group(nx, g, af);
      // Issue order inside the group: the LDS reads of the next group first, then the MFMAs
      // with the refill behind the first of them.
      __builtin_amdgcn_sched_group_barrier(0x100, NC, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, NC * E - 1, 0);
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
  auto park = [&](T* buf, const acc_t (&v)[NC], T sign) {
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) buf[(16 * c + col_of(r)) * LD + row_of(r)] = sign * v[c][r];
  };

  acc_t res[NBLK][NC];
  T af[STEPS];
  auto load_block = [&](int idx) {  // addresses clamped; mask_block zeroes what does not exist
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        long off;
        (void)place(idx, c, r, off);
        res[idx][c][r] = p.B[off];
      }
  };
  auto mask_block = [&](int idx) {
#pragma unroll
    for (int c = 0; c < NC; ++c)
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
      acc_t acc[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[c][r] = T(0);
      product(P, af, acc, nx);
#pragma unroll
      for (int c = 0; c < NC; ++c) res[i][c] = acc[c];
    }
    if (i + 1 < NBLK) {
      // Q was last read by the updates with X_(i-1), which every wave finished before the
      // barrier in front of this leaf.
      park(Q, res[i], T(-1));
      __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < NC; ++c)
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

template <class T, int NBLK, bool SWAP, int NC>
static rtat_status_t launch_panel_as(rtat_native_handle* h, const PanelArgs<T>& a) {
  const size_t lds_bytes = (size_t)2 * PANEL_W * NC * PanelLd<T>::LD * sizeof(T);
  auto kern = trsm_panel_kernel<T, NBLK, SWAP, NC>;
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
  const unsigned grid = (unsigned)((a.nrhs + PANEL_W * NC - 1) / (PANEL_W * NC));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(PANEL_THREADS), lds_bytes, h->stream, a);
  return launch_status();
}

template <class T, int NBLK>
static rtat_status_t launch_panel_n(rtat_native_handle* h, const PanelArgs<T>& a, bool wide) {
  if (wide)
    return a.sp == 1 ? launch_panel_as<T, NBLK, true, 2>(h, a)
                     : launch_panel_as<T, NBLK, false, 2>(h, a);
  return a.sp == 1 ? launch_panel_as<T, NBLK, true, 1>(h, a)
                   : launch_panel_as<T, NBLK, false, 1>(h, a);
}

template <class T>
static rtat_status_t launch_panel(rtat_native_handle* h, const PanelArgs<T>& a, bool wide) {
  static_assert(PANEL_TALL == 8 * NB, "one instantiation per block count of a panel");
  switch ((a.rows + NB - 1) / NB) {
    case 1: return launch_panel_n<T, 1>(h, a, wide);
    case 2: return launch_panel_n<T, 2>(h, a, wide);
    case 3: return launch_panel_n<T, 3>(h, a, wide);
    case 4: return launch_panel_n<T, 4>(h, a, wide);
    case 5: return launch_panel_n<T, 5>(h, a, wide);
    case 6: return launch_panel_n<T, 6>(h, a, wide);
    case 7: return launch_panel_n<T, 7>(h, a, wide);
    case 8: return launch_panel_n<T, 8>(h, a, wide);
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
  bool wide;  // 32 right-hand sides per panel workgroup instead of 16
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
    c.st = launch_panel<T>(c.h, a, c.wide);
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

// Right-hand sides per panel workgroup: 32 (two column tiles) where 16 would give more
// workgroups than the device has CUs, else 16.  Only one workgroup fits a CU, so with 16 a
// second round would start; and with 32 every value of M read from L2 feeds two MFMAs.
static bool wide_panels(const rtat_native_handle* h, int nrhs) {
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  return (nrhs + PANEL_W - 1) / PANEL_W > cus;
}

// Panel height of a call.  The tall panel saves a level of GEMM updates: a 1024-row panel
// runs as fast per block product as a 512-row one, which makes it cheaper than two short
// panels and the 512-deep update between them wherever the panel kernel has workgroups for a
// good part of the machine (measured on MI355X, 8192 right-hand sides: 48 + 68 + 48 us against
// 152 us; DTRSM n = 8192 7.83 -> 7.70 ms, n = 4096 1.21 -> 1.08 ms).  With workgroups for at
// most half the CUs the panel kernel leaves most of the machine idle, and the update it would
// absorb is better off as a GEMM over all CUs.
static int pick_panel(const rtat_native_handle* h, int nrhs) {
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  const long groups = (nrhs + PANEL_W - 1) / PANEL_W;
  return 2 * groups <= cus ? PANEL_SHORT : PANEL_TALL;
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
                                                   : pick_panel(h, left ? n : m);
  h->last.trsm_panel_rows = panel;
  const bool wide = wide_panels(h, left ? n : m);
  h->last.trsm_panel_width = wide ? 2 * PANEL_W : PANEL_W;
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
                     unit ? 1 : 0, mtrans ? 1 : 0, inv, packed, panel / NB);
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
