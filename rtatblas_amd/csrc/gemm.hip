// fp64 DGEMM / DSYRK core for gfx950 on v_mfma_f64_16x16x4_f64.
//
// Serves gpuTgemm and gpuTsyrk of the reference (src/matrix_ops/matrixop.h:15-76), which
// forward to hipblasDgemm / hipblasDsyrk.  Column-major C(m x n) = alpha*op(A)*op(B) + beta*C.
//
// Structure
//   * One workgroup = 4 (or 8) waves = one BM x BN macro tile of C; the K loop advances
//     BK = 16 at a time through two LDS stages: while the MFMAs of stage s run, the next
//     panel pair is already in registers (global -> VGPR prefetch two panels ahead) and is
//     written to the other stage early in the iteration; one barrier per iteration.
//   * Operand panels live in LDS in the orientation they have in global memory, so the
//     global -> LDS copy is a straight vector copy for all four (opA, opB) combinations:
//     "k-major" panels ([row][k], row stride BK+2) for operands contiguous along k, and
//     "mn-major" panels ([k][row], row stride rows+16) for operands contiguous along m / n.
//   * MFMA operands leave LDS as 16-byte reads only.  The MFMA blocks of a wave interleave
//     their rows in pairs and the K-steps interleave their k in pairs (frag_row, frag_k), so
//     that a lane's two values are neighbours in either panel orientation; with the strides
//     above both read patterns and both write patterns are free of bank conflicts.
//   * The MFMA is issued as D^T = B^T A^T: its "A" slot takes the n-side operand and its
//     "B" slot the m-side operand, so that the lane index l%16 of the accumulator runs
//     along m, the contiguous dimension of column-major C; a lane stores two neighbouring
//     rows as one 16-byte access.
//   * Global loads are buffer loads (scalar tile base + 32-bit lane offset).  Rows of a tile
//     that hang over the edge of C are clamped onto the last valid row, so edge tiles run the
//     same loop as interior ones; only the K tail and the last two panels take per-element
//     guarded loads that zero-fill.  Any m, n, k, ld is accepted; odd leading dimensions or
//     unaligned bases fall back from 16-byte to 8-byte loads.
//   * Workgroup ids are remapped so that each of the 8 XCDs (ids are dealt round-robin to
//     XCDs) walks a compact band of tiles and shares panels through its own L2.
//
// Algorithmic work: 2*m*n*k flop (DSYRK: n*(n+1)*k).
#include "common.h"

namespace rtat_native {

typedef double d2_t __attribute__((ext_vector_type(2)));
typedef double d4_t __attribute__((ext_vector_type(4)));
typedef unsigned u2_t __attribute__((ext_vector_type(2)));
typedef unsigned u4_t __attribute__((ext_vector_type(4)));

struct GemmArgs {
  int m, n, k;
  double alpha, beta;
  const double* A;
  long lda;
  const double* B;
  long ldb;
  double* C;
  long ldc;
  int tiles_m, tiles_n;
  int tri;   // 0: full C; 1: lower triangle only; 2: upper triangle only
  int wide;  // 1: a tile of A or B spans 4 GiB or more, the 32-bit-offset loads are off
};

template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int WG_PER_CU_>
struct TileShape {
  static constexpr int WG_PER_CU = WG_PER_CU_;  // occupancy the register budget is set for
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int WGM = WGM_, WGN = WGN_;      // waves along m / n
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;  // wave tile
  static constexpr int TM = WTM / 16, TN = WTN / 16;    // MFMA blocks per wave tile
  static constexpr int NT = 64 * WGM * WGN;                // lanes per workgroup
  static_assert(BK % 8 == 0, "K step splits in two halves of whole MFMA steps");
};

// Panel of ROWS x BK doubles in LDS.
template <bool KMAJOR, int ROWS, int BK>
struct Panel {
  static constexpr int STRIDE = KMAJOR ? BK + 2 : ROWS + 16;
  static constexpr int SIZE = KMAJOR ? ROWS * STRIDE : BK * STRIDE;
  __device__ static inline int off(int row, int k) {
    return KMAJOR ? row * STRIDE + k : k * STRIDE + row;
  }
};

// Row of the 16x16 fp64 MFMA result held in accumulator register r of lane `lane`
// (the column is lane % 16).
__device__ inline int mfma_f64_row(int r, int lane) { return 4 * r + (lane >> 4); }

// Which of the 16*T tile rows MFMA block `blk` takes from operand lane `l16`: blocks come in
// pairs that interleave their rows (block 2p takes the even rows of a 32-row group, block
// 2p+1 the odd ones), so that one lane's rows for a block pair are neighbours.
__device__ inline int frag_row(int blk, int l16) { return 32 * (blk >> 1) + 2 * l16 + (blk & 1); }

// The k index (0 .. BK-1) that lane group kq (lane / 16) feeds to MFMA step `step` of a
// 16-wide panel: steps come in pairs that interleave their k, so that one lane's k for a
// step pair are neighbours.  Any assignment works as long as both operands use the same.
__device__ inline int frag_k(int step, int kq) { return 8 * (step >> 1) + 2 * kq + (step & 1); }

// Operand fragments of one step pair (two MFMA K-steps) for T blocks: f[blk][step & 1].
// Every LDS access is one 16-byte read: a k-major panel yields one block's two k at once,
// an mn-major panel yields a block pair's two rows at once; with the row and k interleave
// above both patterns are free of bank conflicts (64 banks, 16 lanes per cycle grouped as
// lanes 0-7 with 24-31 etc.).
template <bool KMAJOR, class P, int T>
__device__ inline void load_frags(const double* panel, int w0, int pair, int l16, int kq,
                                  double (&f)[T][2]) {
  static_assert(T % 2 == 0, "blocks are handled in pairs");
  if constexpr (KMAJOR) {
#pragma unroll
    for (int b = 0; b < T; ++b) {
      const d2_t v = *reinterpret_cast<const d2_t*>(
          panel + P::off(w0 + frag_row(b, l16), frag_k(2 * pair, kq)));
      f[b][0] = v[0];
      f[b][1] = v[1];
    }
  } else {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int b = 0; b < T; b += 2) {
        const d2_t v = *reinterpret_cast<const d2_t*>(
            panel + P::off(w0 + frag_row(b, l16), frag_k(2 * pair + s, kq)));
        f[b][s] = v[0];
        f[b + 1][s] = v[1];
      }
  }
}

// Global -> register -> LDS mover for one operand panel, NT lanes, VEC doubles per access.
template <bool KMAJOR, int ROWS, int BK, int VEC, int NT>
struct Mover {
  typedef Panel<KMAJOR, ROWS, BK> P;
  static constexpr int NV = ROWS * BK / (VEC * NT);         // accesses per lane per panel
  static constexpr int INNER = (KMAJOR ? BK : ROWS) / VEC;  // vectors along the contiguous dim
  static constexpr int OUTER_STEP = NT / INNER;             // outer index step per pass
  static_assert(NV >= 1 && NT % INNER == 0, "panel must split evenly over the lanes");

  double r[NV][VEC];
  // This lane's byte offsets from the tile's first element: one per pass for a k-major
  // panel (rows are clamped one by one), a single one for an mn-major panel, whose passes
  // step through k by a wave-uniform stride that travels in a scalar register.
  static constexpr int NOFF = KMAJOR ? NV : 1;
  unsigned go[NOFF];

  // Fix the lane's source offsets.  Rows past row_lim are clamped onto the last valid row
  // (they only feed accumulators of C elements that are never stored), so a tile that hangs
  // over the edge of C loads exactly like an interior one.  A 2-vector that runs along the
  // rows starts on an even row; when the valid rows end on an odd count its second element
  // is the first element of the next stored column, which exists for every column but the
  // operand's last: the caller keeps that column out of the vector path.  The launcher
  // guarantees that a tile's footprint fits 32-bit byte offsets before it lets a kernel use
  // this path.
  __device__ inline void init(long ld, int row0, int row_lim, int t) {
    const int in = (t % INNER) * VEC, out = t / INNER;
    if constexpr (KMAJOR) {
#pragma unroll
      for (int p = 0; p < NV; ++p) {
        int row = row0 + out + p * OUTER_STEP;
        row = row < row_lim ? row : row_lim - 1;
        go[p] = (unsigned)(((long)(row - row0) * ld + in) * 8);
      }
    } else {
      const int last = VEC == 2 ? ((row_lim - 1) & ~1) : row_lim - 1;
      int row = row0 + in;
      row = row < last ? row : last;
      go[0] = (unsigned)(((long)out * ld + (row - row0)) * 8);
    }
  }

  // Full panel kt of the tile that starts at row0: every k index in range and, for VEC == 2,
  // every access 16-byte aligned.  Buffer loads: the tile's first element is the (scalar)
  // base of the descriptor, the lane offset a 32-bit register, the pass stride a scalar.
  __device__ inline void load_fast(const double* base, long ld, int row0, int kt) {
    const double* tile =
        KMAJOR ? base + (long)row0 * ld + (long)kt * BK : base + (long)kt * BK * ld + row0;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<double*>(tile), 0, 0xffffffff, 0x00020000);
#pragma unroll
    for (int p = 0; p < NV; ++p) {
      const unsigned voff = KMAJOR ? go[p] : go[0];
      const unsigned soff = KMAJOR ? 0u : (unsigned)((long)(p * OUTER_STEP) * ld * 8);
      if constexpr (VEC == 2) {
        const u4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0);
        const d2_t d = __builtin_bit_cast(d2_t, v);
        r[p][0] = d[0];
        r[p][1] = d[1];
      } else {
        const u2_t v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, soff, 0);
        r[p][0] = __builtin_bit_cast(double, v);
      }
    }
  }

  // Edge panel, element-wise and branch free.  Rows past row_lim are clamped onto the last
  // valid row: they only feed accumulators of C elements that are never stored.  k past
  // k_lim is clamped for the address and the value replaced by zero, because those products
  // would land in valid C elements.
  __device__ inline void load_edge(const double* base, long ld, int row0, int row_lim, int k0,
                                   int k_lim, int t) {
    const int in = (t % INNER) * VEC, out = t / INNER;
#pragma unroll
    for (int p = 0; p < NV; ++p) {
      const int o = out + p * OUTER_STEP;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        int row = KMAJOR ? row0 + o : row0 + in + e;
        int kk = KMAJOR ? k0 + in + e : k0 + o;
        const bool k_ok = kk < k_lim;
        row = row < row_lim ? row : row_lim - 1;
        kk = k_ok ? kk : k_lim - 1;
        const double v = KMAJOR ? base[(long)row * ld + kk] : base[(long)kk * ld + row];
        r[p][e] = k_ok ? v : 0.0;
      }
    }
  }

  __device__ inline void store(double* panel, int t) const {
    const int in = (t % INNER) * VEC, out = t / INNER;
#pragma unroll
    for (int p = 0; p < NV; ++p) {
      const int o = out + p * OUTER_STEP;
      double* s = panel + (KMAJOR ? P::off(o, in) : P::off(in, o));
      if constexpr (VEC == 2) {
        d2_t v;
        v[0] = r[p][0];
        v[1] = r[p][1];
        *reinterpret_cast<d2_t*>(s) = v;
      } else {
        *s = r[p][0];
      }
    }
  }
};

// Scheduling hint: spread NA instructions of class MASK_A and NB of class MASK_B evenly
// behind N MFMAs (one MFMA, then that MFMA's share of the others, and so on).  A 64-cycle
// fp64 MFMA hides only a handful of issue slots, so memory instructions must trail the
// MFMAs one or two at a time; issued as a burst they stall the matrix pipe.
// Classes (LLVM sched_group_barrier masks): 0x008 MFMA, 0x020 VMEM read, 0x100 DS read,
// 0x200 DS write.
template <int I, int N, int NA, int MASK_A, int NB, int MASK_B>
__device__ inline void interleave_behind_mfma() {
  if constexpr (I < N) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    constexpr int a = NA * (I + 1) / N - NA * I / N;
    constexpr int b = NB * (I + 1) / N - NB * I / N;
    if constexpr (a > 0) __builtin_amdgcn_sched_group_barrier(MASK_A, a, 0);
    if constexpr (b > 0) __builtin_amdgcn_sched_group_barrier(MASK_B, b, 0);
    interleave_behind_mfma<I + 1, N, NA, MASK_A, NB, MASK_B>();
  }
}

constexpr int XCDS = 8;
constexpr int BAND = 4;  // tile columns per band of the tile walk

// Tiles of a triangular C (SYRK) that hold at least one element of the wanted triangle, per
// tile row i: lower (tri == 1) keeps columns [0, count), upper (tri == 2) keeps
// [tiles_n - count, tiles_n).  Shared by the launcher (grid size) and the kernel (mapping).
__host__ __device__ inline int tri_row_count(int tri, int i, int bm, int bn, int tiles_n) {
  if (tri == 1) {
    const int c = ((i + 1) * bm - 1) / bn + 1;  // columns with n0 <= m0 + bm - 1
    return c < tiles_n ? c : tiles_n;
  }
  const int first = (i * bm) / bn;  // first column with n0 + bn - 1 >= m0
  return first < tiles_n ? tiles_n - first : 0;
}

// Workgroup id -> (tile row, tile column).  Ids are dealt round-robin to the XCDs, so XCD x
// sees ids x, x+8, ...; give it one contiguous slice of the logical tile order.
//   * Full C: the order walks bands of BAND tile columns, tile columns fastest across a band,
//     so the ~64 tiles an XCD has in flight share few distinct A and B panels; and it is
//     walked backwards, so that the ragged last tile row / column, whose guarded loads are
//     slower, start first instead of forming the tail.
//   * Triangular C: only tiles that touch the triangle are enumerated (row by row), so every
//     XCD gets the same number of real tiles.
__device__ inline void tile_of_workgroup(int wg, int nwg, int tiles_m, int tiles_n, int tri,
                                         int bm, int bn, int& tm, int& tn) {
  const int per = nwg / XCDS, rem = nwg % XCDS;
  const int x = wg % XCDS, i = wg / XCDS;
  int logical = x * per + (x < rem ? x : rem) + i;
  if (tri != 0) {
    int row = 0;
    for (;;) {
      const int c = tri_row_count(tri, row, bm, bn, tiles_n);
      if (logical < c) break;
      logical -= c;
      ++row;
    }
    tm = row;
    tn = (tri == 1) ? logical : tiles_n - tri_row_count(tri, row, bm, bn, tiles_n) + logical;
    return;
  }
  logical = nwg - 1 - logical;
  const int band_tiles = BAND * tiles_m;
  const int band = logical / band_tiles, in = logical % band_tiles;
  const int left = tiles_n - band * BAND;
  const int width = left < BAND ? left : BAND;
  tm = in / width;
  tn = band * BAND + in % width;
}

template <class TS, bool TA, bool TB, int VEC>
__global__ __launch_bounds__(TS::NT, TS::WG_PER_CU) void dgemm_kernel(GemmArgs p) {
  constexpr int BM = TS::BM, BN = TS::BN, BK = TS::BK, TM = TS::TM, TN = TS::TN;
  constexpr bool A_KMAJOR = TA;    // op(A) = A^T: A stored k x m, contiguous along k
  constexpr bool B_KMAJOR = !TB;   // op(B) = B:   B stored k x n, contiguous along k
  typedef Panel<A_KMAJOR, BM, BK> PA;
  typedef Panel<B_KMAJOR, BN, BK> PB;
  constexpr int STAGE = PA::SIZE + PB::SIZE;
  extern __shared__ __align__(16) double lds[];

  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, p.tri, BM, BN, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm0 = (wave % TS::WGM) * TS::WTM, wn0 = (wave / TS::WGM) * TS::WTN;
  const int r16 = lane & 15, kq = lane >> 4;

  const bool interior = (m0 + BM <= p.m) && (n0 + BN <= p.n);
  const int nkt = (p.k + BK - 1) / BK;

  Mover<A_KMAJOR, BM, BK, VEC, TS::NT> mva;
  Mover<B_KMAJOR, BN, BK, VEC, TS::NT> mvb;

  mva.init(p.lda, m0, p.m, t);
  mvb.init(p.ldb, n0, p.n, t);
  auto gload_fast = [&](int kt) {
    mva.load_fast(p.A, p.lda, m0, kt);
    mvb.load_fast(p.B, p.ldb, n0, kt);
  };
  auto gload_edge = [&](int kt) {
    mva.load_edge(p.A, p.lda, m0, p.m, kt * BK, p.k, t);
    mvb.load_edge(p.B, p.ldb, n0, p.n, kt * BK, p.k, t);
  };
  // Panel pair kt is "fast" when it is a full BK; for a tile that hangs over the edge of C it
  // must also stay clear of the operands' last stored column (see Mover::init).
  const int nkt_fast = p.wide ? 0 : (interior ? p.k / BK : (p.k - 1) / BK);
  auto gload = [&](int kt) {
    if (kt < nkt_fast) gload_fast(kt);
    else gload_edge(kt);
  };
  auto lstore = [&](int stage) {
    mva.store(lds + stage * STAGE, t);
    mvb.store(lds + stage * STAGE + PA::SIZE, t);
  };

  d4_t acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) acc[j][i] = d4_t{0.0, 0.0, 0.0, 0.0};

  // Operand fragments: two sets, each holding one step pair (two MFMA K-steps).
  double mf[2][TM][2], nf[2][TN][2];
  auto fetch = [&](int stage, int pair, int set) {
    const double* sa = lds + stage * STAGE;
    load_frags<A_KMAJOR, PA, TM>(sa, wm0, pair, r16, kq, mf[set]);
    load_frags<B_KMAJOR, PB, TN>(sa + PA::SIZE, wn0, pair, r16, kq, nf[set]);
  };
  auto mfma_step = [&](int set, int s) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        acc[j][i] =
            __builtin_amdgcn_mfma_f64_16x16x4f64(nf[set][j][s], mf[set][i][s], acc[j][i], 0, 0, 0);
  };
  static_assert(BK == 16, "the pipeline below is written for four K-steps per stage");

  if (nkt > 0) {
    gload(0);
    lstore(0);
    if (nkt > 1) gload(1);
    __syncthreads();
    // Same issue pattern as the tail of a loop iteration, so that the wait counts the
    // compiler derives at the loop head are the loop's own, not the prologue's.
    __builtin_amdgcn_sched_barrier(0);
    fetch(0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }

  // One iteration = one BK panel pair = four K-steps = two step pairs.  Every memory
  // instruction is issued at least one K-step of MFMAs ahead of its consumer or of the
  // barrier, and trails the MFMAs one instruction at a time:
  //   step 0 (set 0) | park the prefetched panels in the other stage, start the next global
  //                  | prefetch (two panels ahead)
  //   step 1 (set 0) | read the fragments of steps 2 and 3 (set 1)
  //   barrier          (writes and reads were issued a K-step ago: only wave skew is left)
  //   step 2 (set 1) | read steps 0 and 1 of the NEXT stage (set 0)
  //   step 3 (set 1) |
  // Full panels run the first loop, whose prefetch is the unguarded vector load and whose
  // body is one basic block per phase; the K tail and the last two panels run the second,
  // guarded loop.
  constexpr int NMFMA = TM * TN;
  constexpr int NMOVE = decltype(mva)::NV + decltype(mvb)::NV;  // global loads = LDS stores
  constexpr int NFRAG = TM + TN;                                // LDS reads per step pair
  int kt = 0;
  for (; kt + 2 < nkt_fast; ++kt) {
    const int cur = kt & 1, nxt = cur ^ 1;
    mfma_step(0, 0);
    lstore(nxt);
    gload_fast(kt + 2);
    interleave_behind_mfma<0, NMFMA, NMOVE, 0x200, NMOVE, 0x020>();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(0, 1);
    fetch(cur, 1, 1);
    interleave_behind_mfma<0, NMFMA, NFRAG, 0x100, 0, 0>();
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(1, 0);
    fetch(nxt, 0, 0);
    interleave_behind_mfma<0, NMFMA, NFRAG, 0x100, 0, 0>();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(1, 1);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (; kt + 1 < nkt; ++kt) {
    const int cur = kt & 1, nxt = cur ^ 1;
    mfma_step(0, 0);
    lstore(nxt);
    gload(kt + 2 < nkt ? kt + 2 : nkt - 1);
    __builtin_amdgcn_sched_barrier(0);
    fetch(cur, 1, 1);
    mfma_step(0, 1);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(1, 0);
    fetch(nxt, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(1, 1);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (nkt > 0) {
    const int cur = (nkt - 1) & 1;
    fetch(cur, 1, 1);
    mfma_step(0, 0);
    mfma_step(0, 1);
    mfma_step(1, 0);
    mfma_step(1, 1);
  }

  // Epilogue.  Accumulator (j, i), register r, lane l  ->  C(row, col) with
  // row = m0 + wm0 + frag_row(i, l % 16), col = n0 + wn0 + frag_row(j, mfma_f64_row(r, l)).
  // Blocks i and i+1 hold neighbouring rows, so a lane stores them as one 16-byte pair
  // when C allows it (even ldc on a 16-byte aligned base; row pairs start on even rows).
  const double alpha = p.alpha, beta = p.beta;
  const bool pair_ok = ((p.ldc & 1) == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 15u) == 0);
#pragma unroll
  for (int j = 0; j < TN; ++j) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int col = n0 + wn0 + frag_row(j, mfma_f64_row(r, lane));
      if (col >= p.n) continue;
      double* ccol = p.C + (long)col * p.ldc;
#pragma unroll
      for (int i = 0; i < TM; i += 2) {
        const int row = m0 + wm0 + frag_row(i, r16);
        if (row >= p.m) continue;
        const bool both = row + 1 < p.m;
        bool keep0 = true, keep1 = both;
        if (p.tri == 1) { keep0 = row >= col; keep1 = keep1 && row + 1 >= col; }
        if (p.tri == 2) { keep0 = row <= col; keep1 = keep1 && row + 1 <= col; }
        double v0 = alpha * acc[j][i][r], v1 = alpha * acc[j][i + 1][r];
        if (pair_ok && keep0 && keep1) {
          d2_t* c2 = reinterpret_cast<d2_t*>(ccol + row);
          if (beta != 0.0) {
            const d2_t old = *c2;
            v0 += beta * old[0];
            v1 += beta * old[1];
          }
          d2_t out;
          out[0] = v0;
          out[1] = v1;
          *c2 = out;
        } else {
          if (keep0) {
            if (beta != 0.0) v0 += beta * ccol[row];
            ccol[row] = v0;
          }
          if (keep1) {
            if (beta != 0.0) v1 += beta * ccol[row + 1];
            ccol[row + 1] = v1;
          }
        }
      }
    }
  }
}

// C = beta*C on one triangle (or all) of C: the alpha == 0 / k == 0 case.
__global__ __launch_bounds__(256) void scale_c_kernel(int m, int n, double beta, double* C,
                                                     long ldc, int tri) {
  const int row = blockIdx.x * 256 + threadIdx.x;
  if (row >= m) return;
  for (int col = blockIdx.y; col < n; col += gridDim.y) {
    if (tri == 1 && row < col) continue;
    if (tri == 2 && row > col) continue;
    double* c = C + row + (long)col * ldc;
    *c = (beta == 0.0) ? 0.0 : beta * *c;
  }
}

template <class TS, bool TA, bool TB, int VEC>
static rtat_status_t launch_tile(rtat_native_handle* h, const GemmArgs& a) {
  typedef Panel<TA, TS::BM, TS::BK> PA;
  typedef Panel<!TB, TS::BN, TS::BK> PB;
  const size_t lds_bytes = 2 * (size_t)(PA::SIZE + PB::SIZE) * sizeof(double);
  auto kern = dgemm_kernel<TS, TA, TB, VEC>;
  static bool configured = false;
  if (!configured) {
    if (lds_bytes > 65536 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess) {
      (void)hipGetLastError();
      return RTAT_STATUS_NOT_SUPPORTED;
    }
    configured = true;
  }
  GemmArgs p = a;
  // Bytes from a tile's first element to its farthest one, per operand.
  const long span_a = TA ? ((long)(TS::BM - 1) * a.lda + TS::BK) * 8
                         : ((long)(TS::BK - 1) * a.lda + TS::BM) * 8;
  const long span_b = !TB ? ((long)(TS::BN - 1) * a.ldb + TS::BK) * 8
                          : ((long)(TS::BK - 1) * a.ldb + TS::BN) * 8;
  p.wide = (span_a >= (1L << 32) || span_b >= (1L << 32)) ? 1 : 0;
  p.tiles_m = (a.m + TS::BM - 1) / TS::BM;
  p.tiles_n = (a.n + TS::BN - 1) / TS::BN;
  long nwg = (long)p.tiles_m * p.tiles_n;
  if (a.tri != 0) {
    nwg = 0;
    for (int i = 0; i < p.tiles_m; ++i) nwg += tri_row_count(a.tri, i, TS::BM, TS::BN, p.tiles_n);
  }
  if (nwg > 0x7fffffffL) return RTAT_STATUS_INVALID_VALUE;
  if (nwg == 0) return RTAT_STATUS_SUCCESS;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(TS::NT), lds_bytes, h->stream, p);
  return launch_status();
}

template <class TS>
static rtat_status_t launch_ops(rtat_native_handle* h, bool ta, bool tb, bool vec,
                                const GemmArgs& a) {
  if (vec) {
    if (!ta && !tb) return launch_tile<TS, false, false, 2>(h, a);
    if (!ta && tb) return launch_tile<TS, false, true, 2>(h, a);
    if (ta && !tb) return launch_tile<TS, true, false, 2>(h, a);
    return launch_tile<TS, true, true, 2>(h, a);
  }
  if (!ta && !tb) return launch_tile<TS, false, false, 1>(h, a);
  if (!ta && tb) return launch_tile<TS, false, true, 1>(h, a);
  if (ta && !tb) return launch_tile<TS, true, false, 1>(h, a);
  return launch_tile<TS, true, true, 1>(h, a);
}

typedef TileShape<256, 128, 16, 4, 2, 1> T256x128;  // 8 waves of 64x64
typedef TileShape<128, 128, 16, 2, 2, 2> T128x128;  // 4 waves of 64x64, two workgroups per CU
typedef TileShape<128, 64, 16, 2, 2, 2> T128x64;    // 4 waves of 64x32
typedef TileShape<64, 64, 16, 2, 2, 4> T64x64;      // 4 waves of 32x32, four workgroups per CU

// Shape heuristic for RTAT_GEMM_AUTO.  Tiles are dealt evenly to the CUs, so a launch lasts
// about ceil(tiles / CUs) x (tile area) x (k / rate + fixed), where rate is the shape's
// measured steady-state rate relative to 128x128 and `fixed` the prologue and epilogue of a
// tile in units of k.  A CU that ends up with a single resident workgroup has nothing to run
// while that workgroup sits in its barrier, prologue or epilogue: its rate drops a little and
// the fixed part is fully exposed.  Constants fitted on MI355X (n = 2048 .. 8192, k up to 32768).
static int pick_variant(const rtat_native_handle* h, int m, int n, int k, int tri) {
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  struct Cand { int id, bm, bn, per_cu; double rate; };
  const Cand cands[] = {{RTAT_GEMM_T128x128, 128, 128, 2, 1.0},
                        {RTAT_GEMM_T256x128, 256, 128, 1, 0.99},
                        {RTAT_GEMM_T128x64, 128, 64, 2, 0.965},
                        {RTAT_GEMM_T64x64, 64, 64, 4, 0.93}};
  int best = RTAT_GEMM_T128x128;
  double best_cost = 0.0;
  for (const Cand& c : cands) {
    const int tm = (m + c.bm - 1) / c.bm, tn = (n + c.bn - 1) / c.bn;
    long tiles = (long)tm * tn;
    if (tri != 0) {
      tiles = 0;
      for (int i = 0; i < tm; ++i) tiles += tri_row_count(tri, i, c.bm, c.bn, tn);
    }
    const long per_cu = (tiles + cus - 1) / cus;
    const bool lone = per_cu < 2 && c.per_cu > 1;
    const double per_tile = (double)k / (c.rate * (lone ? 0.975 : 1.0)) + (lone ? 400.0 : 230.0);
    const double cost = (double)per_cu * c.bm * c.bn * per_tile;
    if (best_cost == 0.0 || cost < best_cost) {
      best_cost = cost;
      best = c.id;
    }
  }
  return best;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

rtat_status_t launch_dgemm(rtat_native_handle* h, bool ta, bool tb, int m, int n, int k,
                           double alpha, const double* A, int lda, const double* B, int ldb,
                           double beta, double* C, int ldc, int tri, int variant) {
  if (m < 0 || n < 0 || k < 0) return RTAT_STATUS_INVALID_VALUE;
  if (variant < 0 || variant >= RTAT_GEMM_VARIANT_COUNT) return RTAT_STATUS_INVALID_VALUE;
  if (ldc < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (C == nullptr) return RTAT_STATUS_INVALID_VALUE;
  if (alpha == 0.0 || k == 0) {
    if (beta == 1.0) return RTAT_STATUS_SUCCESS;
    dim3 grid((m + 255) / 256, (unsigned)(n > 65535 ? 65535 : n));
    hipLaunchKernelGGL(scale_c_kernel, grid, dim3(256), 0, h->stream, m, n, beta, C, (long)ldc,
                       tri);
    return launch_status();
  }
  const int a_rows = ta ? k : m, b_rows = tb ? n : k;
  if (A == nullptr || B == nullptr || lda < (a_rows > 1 ? a_rows : 1) ||
      ldb < (b_rows > 1 ? b_rows : 1))
    return RTAT_STATUS_INVALID_VALUE;

  GemmArgs a;
  a.m = m; a.n = n; a.k = k;
  a.alpha = alpha; a.beta = beta;
  a.A = A; a.lda = lda; a.B = B; a.ldb = ldb; a.C = C; a.ldc = ldc;
  a.tiles_m = a.tiles_n = 0;
  a.tri = tri;
  a.wide = 0;
  // 16-byte vector loads need even leading dimensions on 16-byte aligned bases.
  const bool vec = aligned16(A) && aligned16(B) && (lda % 2 == 0) && (ldb % 2 == 0);
  if (variant == RTAT_GEMM_AUTO) variant = pick_variant(h, m, n, k, tri);
  switch (variant) {
    case RTAT_GEMM_T256x128: return launch_ops<T256x128>(h, ta, tb, vec, a);
    case RTAT_GEMM_T128x128: return launch_ops<T128x128>(h, ta, tb, vec, a);
    case RTAT_GEMM_T128x64: return launch_ops<T128x64>(h, ta, tb, vec, a);
    default: return launch_ops<T64x64>(h, ta, tb, vec, a);
  }
}

}  // namespace rtat_native
