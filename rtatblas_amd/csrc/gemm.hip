// GEMM / SYRK core for gfx950 on v_mfma_f64_16x16x4_f64 (double) and v_mfma_f32_16x16x4_f32
// (float); one template serves both, sized in 16-byte vectors (2 doubles / 4 floats).
//
// Serves gpuTgemm and gpuTsyrk of the reference (src/matrix_ops/matrixop.h:15-76), which
// forward to hipblas{D,S}gemm / hipblas{D,S}syrk.  Column-major
// C(m x n) = alpha*op(A)*op(B) + beta*C.
//
// Structure
//   * One workgroup = 4 (or 8) waves = one BM x BN macro tile of C; the K loop advances
//     BK = 16 doubles / 32 floats (128 bytes) at a time through two LDS stages: while the
//     MFMAs of stage s run, the next panel pair is already in registers (global -> VGPR
//     prefetch two panels ahead) and is written to the other stage early in the iteration;
//     one barrier per iteration.  Macro tiles: 256 x 128, 128 x 128, 128 x 64, 64 x 64 (the
//     callable variants) and 32 x 32, which only the automatic choice uses, for small problems.
//   * Operand panels live in LDS in the orientation they have in global memory, so the
//     global -> LDS copy is a straight vector copy for all four (opA, opB) combinations:
//     "k-major" panels ([row][k], row stride BK + one vector) for operands contiguous along k, and
//     "mn-major" panels ([k][row], row stride rows+16) for operands contiguous along m / n.
//   * MFMA operands leave LDS as 16-byte reads.  The MFMA blocks of a wave interleave their
//     rows in groups and the K-steps interleave their k in groups (frag_row, frag_k), so that
//     the values one lane needs are neighbours in either panel orientation; with the strides
//     above the read and write patterns are free of bank conflicts.
//   * The MFMA is issued as D^T = B^T A^T: its "A" slot takes the n-side operand and its
//     "B" slot the m-side operand, so that the lane index l%16 of the accumulator runs
//     along m, the contiguous dimension of column-major C; a lane stores two neighbouring
//     rows as one 16-byte access.
//   * Global loads are buffer loads (scalar tile base + 32-bit lane offset).  Rows of a tile
//     that hang over the edge of C are clamped onto the last valid row, so edge tiles run the
//     same loop as interior ones; only the K tail and the last two panels take per-element
//     guarded loads that zero-fill.  Any m, n, k, ld is accepted: the 16-byte buffer loads need
//     element alignment only, so odd leading dimensions take the same path.
//   * A tile that hangs far over the edge of C skips the MFMA blocks without an element of C
//     (launches of several rounds only); whole tiles store C with nontemporal 16-byte stores.
//   * Workgroup ids are remapped so that each of the 8 XCDs (ids are dealt round-robin to
//     XCDs) walks a compact band of tiles and shares panels through its own L2.
//   * Tail splitting: the tiles left over after the last full round of resident workgroups
//     are cut along K into as many slices as fill the machine once more (in a problem of less
//     than one round some tiles get one slice more, so that no slot stays empty); the slices
//     park raw sums in scratch owned by the handle and a small second kernel adds them in a
//     fixed order (deterministic) and applies alpha, beta and the store masks.  The same
//     serves a leftover of more than half a round in which up to half of the CUs hold one
//     tile more than the rest (only those tiles are cut), and problems of less than a round
//     of the smallest shape that would load the CUs unevenly or leave many of them idle.
//   * Tail subdivision: a leftover too large for K slices but well short of a round is
//     computed as 64 x 64 pieces by a second launch, which spreads it evenly over the CUs.
//
// Algorithmic work: 2*m*n*k flop (DSYRK: n*(n+1)*k).
#include "common.h"
#include "gemm_plan.h"
#include "mfma.h"

#include <type_traits>

namespace rtat_native {

template <class T>
struct GemmArgs {
  int m, n, k;
  T alpha, beta;
  const T* A;
  long lda;
  const T* B;
  long ldb;
  T* C;
  long ldc;
  int tiles_m, tiles_n;
  int tri;   // 0: full C; 1: lower triangle only; 2: upper triangle only
  int wide;  // 1: a tile of A or B spans 4 GiB or more, the 32-bit-offset loads are off
  // Tail splitting: the last split_tiles tiles of the logical tile order are each computed by
  // several workgroups, one per slice of the K panels: split_s slices, one more for the last
  // split_more of those tiles (so that the slices can fill the workgroup slots exactly; the
  // tiles with the longer slices come first).  The slices park their raw sums in split_ws
  // ([slice of all sliced tiles in order][BN][BM]); reduce_kernel then finishes those tiles.
  int split_tiles, split_s, split_more;
  T* split_ws;
  // Tail subdivision (a launch of a smaller tile shape over the last tiles of a larger
  // one): the workgroups cover big tiles sub_base .. sub_base + sub_count - 1 of the logical
  // order of sub_bm x sub_bn tiles (tiles_m, tiles_n count those), each cut into this
  // kernel's own tiles.  sub_count == 0: an ordinary launch.
  int sub_base, sub_count, sub_bm, sub_bn;
  // 1: tiles that hang far over the edge of C skip their empty MFMA blocks (see gemm_kernel).
  int mask_thin;
};

template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int WG_PER_CU_>
struct TileShape {
  static constexpr int WG_PER_CU = WG_PER_CU_;  // occupancy the register budget is set for
  static constexpr int BM = BM_, BN = BN_, BK = BK_;
  static constexpr int WGM = WGM_, WGN = WGN_;      // waves along m / n
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;  // wave tile
  static constexpr int TM = WTM / 16, TN = WTN / 16;    // MFMA blocks per wave tile
  static constexpr int NT = 64 * WGM * WGN;                // lanes per workgroup
};

// Panel of ROWS x BK elements in LDS.  Both strides are whole 16-byte vectors; the k-major
// one is 144 bytes and the mn-major one a multiple of 64 bytes plus 64, which is what keeps
// the fragment reads below off each other's banks.
template <class T, bool KMAJOR, int ROWS, int BK>
struct Panel {
  static constexpr int STRIDE = KMAJOR ? BK + Elem<T>::E : ROWS + 16;
  static constexpr int SIZE = KMAJOR ? ROWS * STRIDE : BK * STRIDE;
  __device__ static inline int off(int row, int k) {
    return KMAJOR ? row * STRIDE + k : k * STRIDE + row;
  }
};

// Which of the 16*T tile rows MFMA block `blk` takes from operand lane `l16`: blocks come in
// groups of G that interleave their rows (block G*p + q takes rows q, q + G, ... of a 16*G row
// group), so that one lane's rows for a block group are neighbours.
template <int G>
__device__ inline int frag_row(int blk, int l16) {
  return 16 * G * (blk / G) + G * l16 + blk % G;
}

// The k index (0 .. BK-1) that lane group kq (lane / 16) feeds to MFMA step `step` of a
// panel: steps come in groups of E that interleave their k, so that one lane's k for a step
// group are neighbours.  Any assignment works as long as both operands use the same.
template <int E>
__device__ inline int frag_k(int step, int kq) {
  return 4 * E * (step / E) + E * kq + step % E;
}

// Element g of a vector of the VecOf family, whose one-element member is a plain scalar.
template <class V>
__device__ inline auto vget(const V& v, int g) {
  if constexpr (std::is_arithmetic_v<V>) return v;
  else return v[g];
}
template <class V, class S>
__device__ inline void vset(V& v, int g, S x) {
  if constexpr (std::is_arithmetic_v<V>) v = x;
  else v[g] = x;
}

// Row interleave of an operand with T blocks per wave: a k-major panel is read one row at a
// time, where pairs give the conflict-free lane stride; an mn-major panel is read along the
// rows, a whole vector of them when the block count allows, else a pair.  A wave with a single
// block has nothing to interleave.
template <class T, bool KMAJOR, int TBLK>
struct RowGroup {
  static constexpr int G =
      TBLK == 1 ? 1 : (KMAJOR ? 2 : (TBLK % Elem<T>::E == 0 ? Elem<T>::E : 2));
  static_assert(TBLK % G == 0, "blocks are handled in groups");
};

// Operand fragments of one step group (E MFMA K-steps) for TBLK blocks: f[blk][step % E].
// A k-major panel yields one block's E k values per 16-byte read, an mn-major panel a block
// group's G rows per read.
template <class T, bool KMAJOR, class P, int TBLK>
__device__ inline void load_frags(const T* panel, int w0, int group, int l16, int kq,
                                  T (&f)[TBLK][Elem<T>::E]) {
  constexpr int E = Elem<T>::E, G = RowGroup<T, KMAJOR, TBLK>::G;
  if constexpr (KMAJOR) {
    typedef typename VecOf<T, E>::type vec_t;
#pragma unroll
    for (int b = 0; b < TBLK; ++b) {
      const vec_t v = *reinterpret_cast<const vec_t*>(
          panel + P::off(w0 + frag_row<G>(b, l16), frag_k<E>(E * group, kq)));
#pragma unroll
      for (int s = 0; s < E; ++s) f[b][s] = v[s];
    }
  } else {
    typedef typename VecOf<T, G>::type vec_t;
#pragma unroll
    for (int s = 0; s < E; ++s)
#pragma unroll
      for (int b = 0; b < TBLK; b += G) {
        const vec_t v = *reinterpret_cast<const vec_t*>(
            panel + P::off(w0 + frag_row<G>(b, l16), frag_k<E>(E * group + s, kq)));
#pragma unroll
        for (int g = 0; g < G; ++g) f[b + g][s] = vget(v, g);
      }
  }
}

// Global -> register -> LDS mover for one operand panel, NT lanes, VEC elements per access
// (a whole 16-byte vector, or 1).
template <class T, bool KMAJOR, int ROWS, int BK, int VEC, int NT>
struct Mover {
  typedef Panel<T, KMAJOR, ROWS, BK> P;
  typedef typename VecOf<T, VEC>::type vec_t;
  static constexpr int NV = ROWS * BK / (VEC * NT);         // accesses per lane per panel
  static constexpr int INNER = (KMAJOR ? BK : ROWS) / VEC;  // vectors along the contiguous dim
  static constexpr int OUTER_STEP = NT / INNER;             // outer index step per pass
  static_assert(NV >= 1 && NT % INNER == 0, "panel must split evenly over the lanes");
  static_assert(VEC == 1 || VEC * sizeof(T) == 16, "vector accesses are 16 bytes");

  T r[NV][VEC];
  // This lane's byte offsets from the tile's first element: one per pass for a k-major
  // panel (rows are clamped one by one), a single one for an mn-major panel, whose passes
  // step through k by a wave-uniform stride that travels in a scalar register.
  static constexpr int NOFF = KMAJOR ? NV : 1;
  unsigned go[NOFF];

  // Fix the lane's source offsets.  Rows past row_lim are clamped onto the last valid row
  // (they only feed accumulators of C elements that are never stored), so a tile that hangs
  // over the edge of C loads exactly like an interior one.  A vector that runs along the
  // rows starts on a multiple of VEC; when the valid rows end inside it, its tail holds the
  // first elements of the next stored column, which exist for every column but the
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
        go[p] = (unsigned)(((long)(row - row0) * ld + in) * (long)sizeof(T));
      }
    } else {
      const int last = (row_lim - 1) & ~(VEC - 1);
      int row = row0 + in;
      row = row < last ? row : last;
      go[0] = (unsigned)(((long)out * ld + (row - row0)) * (long)sizeof(T));
    }
  }

  // Full panel kt of the tile that starts at row0: every k index in range and, for VEC > 1,
  // every access 16-byte aligned.  Buffer loads: the tile's first element is the (scalar)
  // base of the descriptor, the lane offset a 32-bit register, the pass stride a scalar.
  __device__ inline void load_fast(const T* base, long ld, int row0, int kt) {
    const T* tile =
        KMAJOR ? base + (long)row0 * ld + (long)kt * BK : base + (long)kt * BK * ld + row0;
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(tile), 0, 0xffffffff, 0x00020000);
#pragma unroll
    for (int p = 0; p < NV; ++p) {
      const unsigned voff = KMAJOR ? go[p] : go[0];
      const unsigned soff =
          KMAJOR ? 0u : (unsigned)((long)(p * OUTER_STEP) * ld * (long)sizeof(T));
      if constexpr (VEC > 1) {
        const u4_t raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0);
        const vec_t v = __builtin_bit_cast(vec_t, raw);
#pragma unroll
        for (int e = 0; e < VEC; ++e) r[p][e] = v[e];
      } else if constexpr (sizeof(T) == 8) {
        const u2_t raw = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, soff, 0);
        r[p][0] = __builtin_bit_cast(T, raw);
      } else {
        const unsigned raw = __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, soff, 0);
        r[p][0] = __builtin_bit_cast(T, raw);
      }
    }
  }

  // Edge panel, element-wise and branch free.  Rows past row_lim are clamped onto the last
  // valid row: they only feed accumulators of C elements that are never stored.  k past
  // k_lim is clamped for the address and the value replaced by zero, because those products
  // would land in valid C elements.
  __device__ inline void load_edge(const T* base, long ld, int row0, int row_lim, int k0,
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
        const T v = KMAJOR ? base[(long)row * ld + kk] : base[(long)kk * ld + row];
        r[p][e] = k_ok ? v : T(0);
      }
    }
  }

  __device__ inline void store(T* panel, int t) const {
    const int in = (t % INNER) * VEC, out = t / INNER;
#pragma unroll
    for (int p = 0; p < NV; ++p) {
      const int o = out + p * OUTER_STEP;
      T* s = panel + (KMAJOR ? P::off(o, in) : P::off(in, o));
      if constexpr (VEC > 1) {
        vec_t v;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = r[p][e];
        *reinterpret_cast<vec_t*>(s) = v;
      } else {
        *s = r[p][0];
      }
    }
  }
};

template <class T, class TS, bool TA, bool TB, int VEC>
__global__ __launch_bounds__(TS::NT, TS::WG_PER_CU) void gemm_kernel(GemmArgs<T> p) {
  constexpr int BM = TS::BM, BN = TS::BN, BK = TS::BK, TM = TS::TM, TN = TS::TN;
  constexpr int E = Elem<T>::E;
  static_assert(BK == 8 * E, "a panel is two step groups of E MFMA K-steps");
  static_assert(BM % BN == 0, "the triangular tile order counts on whole tile columns per row");
  constexpr bool A_KMAJOR = TA;    // op(A) = A^T: A stored k x m, contiguous along k
  constexpr bool B_KMAJOR = !TB;   // op(B) = B:   B stored k x n, contiguous along k
  typedef Panel<T, A_KMAJOR, BM, BK> PA;
  typedef Panel<T, B_KMAJOR, BN, BK> PB;
  typedef typename Elem<T>::acc_t acc_t;
  constexpr int GA = RowGroup<T, A_KMAJOR, TM>::G, GB = RowGroup<T, B_KMAJOR, TN>::G;
  constexpr int STAGE = PA::SIZE + PB::SIZE;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  // Whole tiles first; then the sliced tiles, consecutive workgroups per tile.
  const int whole = (int)gridDim.x - (p.split_tiles * p.split_s + p.split_more);
  const bool sliced = (int)blockIdx.x >= whole;
  int logical = 0, slice = 0, slices = 1, m0, n0;
  long slot_index = 0;
  if (p.sub_count > 0) {
    // Tail subdivision: the pieces of one big tile go to one XCD (ids x, x + 8, ...), so
    // that they share its panels through that XCD's L2.
    const int pieces_m = p.sub_bm / BM, pieces = pieces_m * (p.sub_bn / BN);
    const int x = (int)blockIdx.x % XCDS, j = (int)blockIdx.x / XCDS;
    const int big = (j / pieces) * XCDS + x, piece = j % pieces;
    if (big >= p.sub_count) return;
    int big_m, big_n;
    tile_of_logical(p.sub_base + big, p.tiles_m, p.tiles_n, p.tri, p.sub_bm, p.sub_bn, big_m,
                    big_n);
    m0 = big_m * p.sub_bm + (piece % pieces_m) * BM;
    n0 = big_n * p.sub_bn + (piece / pieces_m) * BN;
    // Pieces past the edge of C, or wholly outside the wanted triangle, have nothing to do.
    if (m0 >= p.m || n0 >= p.n) return;
    if (p.tri == 1 && m0 + BM - 1 < n0) return;
    if (p.tri == 2 && m0 > n0 + BN - 1) return;
  } else {
    if (!sliced) {
      logical = logical_of_workgroup(blockIdx.x, whole);
    } else {
      const int idx = (int)blockIdx.x - whole;
      const int plain_wgs = (p.split_tiles - p.split_more) * p.split_s;
      int tile;
      if (idx < plain_wgs) {
        slices = p.split_s;
        tile = idx / slices;
        slice = idx % slices;
      } else {
        slices = p.split_s + 1;
        tile = p.split_tiles - p.split_more + (idx - plain_wgs) / slices;
        slice = (idx - plain_wgs) % slices;
      }
      logical = whole + tile;
      slot_index = idx;
    }
    int tile_m, tile_n;
    tile_of_logical(logical, p.tiles_m, p.tiles_n, p.tri, BM, BN, tile_m, tile_n);
    m0 = tile_m * BM;
    n0 = tile_n * BN;
  }

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm0 = (wave % TS::WGM) * TS::WTM, wn0 = (wave / TS::WGM) * TS::WTN;
  const int r16 = lane & 15, kq = lane >> 4;

  // The K range of this workgroup: all of it, or one slice of whole panels (the last slice
  // also takes the ragged end).  A and B are advanced to the slice's first panel.
  int kbeg = 0, klen = p.k;
  if (sliced) {  // panels [slice * n / slices, (slice + 1) * n / slices) of the n K panels
    const long panels = (p.k + BK - 1) / BK;
    kbeg = (int)(slice * panels / slices) * BK;
    const int kend = (slice == slices - 1) ? p.k : (int)((slice + 1) * panels / slices) * BK;
    klen = kend - kbeg;
  }
  const bool to_k_end = kbeg + klen == p.k;
  const T* Ap = A_KMAJOR ? p.A + kbeg : p.A + (long)kbeg * p.lda;
  const T* Bp = B_KMAJOR ? p.B + kbeg : p.B + (long)kbeg * p.ldb;

  const bool interior = (m0 + BM <= p.m) && (n0 + BN <= p.n);
  const int nkt = (klen + BK - 1) / BK;

  Mover<T, A_KMAJOR, BM, BK, VEC, TS::NT> mva;
  Mover<T, B_KMAJOR, BN, BK, VEC, TS::NT> mvb;

  mva.init(p.lda, m0, p.m, t);
  mvb.init(p.ldb, n0, p.n, t);
  auto gload_fast = [&](int kt) {
    mva.load_fast(Ap, p.lda, m0, kt);
    mvb.load_fast(Bp, p.ldb, n0, kt);
  };
  auto gload_edge = [&](int kt) {
    mva.load_edge(Ap, p.lda, m0, p.m, kt * BK, klen, t);
    mvb.load_edge(Bp, p.ldb, n0, p.n, kt * BK, klen, t);
  };
  // Panel pair kt is "fast" when it is a full BK; for a tile that hangs over the edge of C it
  // must also stay clear of the operands' last stored column (see Mover::init).
  const int nkt_fast = p.wide ? 0 : ((interior || !to_k_end) ? klen / BK : (klen - 1) / BK);
  auto gload = [&](int kt) {
    if (kt < nkt_fast) gload_fast(kt);
    else gload_edge(kt);
  };
  auto lstore = [&](int stage) {
    mva.store(lds + stage * STAGE, t);
    mvb.store(lds + stage * STAGE + PA::SIZE, t);
  };

  acc_t acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[j][i][r] = T(0);

  // Operand fragments: two sets, each holding one step group (E MFMA K-steps).
  T mf[2][TM][E], nf[2][TN][E];
  auto fetch = [&](int stage, int group, int set) {
    const T* sa = lds + stage * STAGE;
    load_frags<T, A_KMAJOR, PA, TM>(sa, wm0, group, r16, kq, mf[set]);
    load_frags<T, B_KMAJOR, PB, TN>(sa + PA::SIZE, wn0, group, r16, kq, nf[set]);
  };
  auto mfma_step = [&](int set, int s) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        acc[j][i] = Elem<T>::mfma(nf[set][j][s], mf[set][i][s], acc[j][i]);
  };
  // Thin tiles.  A tile of which a quarter or more of the rows or columns hangs over the edge
  // of C leaves out the MFMA blocks that hold no element of C: bit j * TM + i of `live` says
  // whether this wave's block (j, i) has one.  The decision is the workgroup's (all waves run
  // the same loop), the mask the wave's; a wave without live blocks still moves its share of
  // the panels.  Such a tile runs the guarded loop, whose iterations are bound by the latency
  // of the panel loads rather than by the matrix pipe: that frees the pipe for the workgroup
  // it shares the CU with, but on a CU of its own it is slower than the plain loop, so the
  // launcher allows it only in launches of several rounds (p.mask_thin; 8200 x 8200 x 4096 NT
  // 7734 -> 7518 us, 4097^3 TN 1980 -> 1955 us; in the single round of 1000^3 it would cost
  // 37.6 -> 51.9 us).
  static_assert(TM * TN <= 32, "one bit per MFMA block of a wave");
  const int rows_in = p.m - m0, cols_in = p.n - n0;
  const bool thin = p.mask_thin != 0 && (rows_in * 4 <= BM * 3 || cols_in * 4 <= BN * 3);
  unsigned live = ~0u;
  if (thin) {
    live = 0u;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        if (wm0 + frag_row<GA>(i, 0) < rows_in && wn0 + frag_row<GB>(j, 0) < cols_in)
          live |= 1u << (j * TM + i);
    live = __builtin_amdgcn_readfirstlane(live);
  }
  auto mfma_live = [&](int set, int s) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        if ((live >> (j * TM + i)) & 1u)
          acc[j][i] = Elem<T>::mfma(nf[set][j][s], mf[set][i][s], acc[j][i]);
  };

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

  // One iteration = one BK panel pair = two step groups of E K-steps.  Every memory
  // instruction is issued at least one K-step of MFMAs ahead of its consumer or of the
  // barrier, and trails the MFMAs one instruction at a time:
  //   group 0, step 0 (set 0) | park the prefetched panels in the other stage, start the next
  //                           | global prefetch (two panels ahead)
  //   group 0, step 1 (set 0) | read the fragments of group 1 (set 1)
  //   group 0, further steps
  //   barrier          (writes and reads were issued a K-step ago: only wave skew is left)
  //   group 1, step 0 (set 1) | read group 0 of the NEXT stage (set 0)
  //   group 1, further steps
  // Full panels run the first loop, whose prefetch is the unguarded vector load and whose
  // body is one basic block per phase; a K tail (and the two panels before it) runs the
  // second, guarded loop, and so does a thin tile from its first panel on.
  constexpr int NMFMA = TM * TN;
  constexpr int NMOVE = decltype(mva)::NV + decltype(mvb)::NV;  // global loads = LDS stores
  constexpr int NFRAG = (A_KMAJOR ? TM : E * TM / GA) + (B_KMAJOR ? TN : E * TN / GB);
  // When every panel is a full one the first loop also runs the last iterations, whose
  // prefetch index is clamped (the last panel is fetched again and never used).
  int kt = 0;
  const int fast_end = thin ? 0 : (nkt_fast == nkt ? nkt - 1 : nkt_fast - 2);
  for (; kt < fast_end; ++kt) {
    const int cur = kt & 1, nxt = cur ^ 1;
    mfma_step(0, 0);
    lstore(nxt);
    gload_fast(kt + 2 < nkt ? kt + 2 : nkt - 1);
    interleave_behind_mfma<0, NMFMA, NMOVE, 0x200, NMOVE, 0x020>();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(0, 1);
    fetch(cur, 1, 1);
    interleave_behind_mfma<0, NMFMA, NFRAG, 0x100, 0, 0>();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 2; s < E; ++s) {
      mfma_step(0, s);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(1, 0);
    fetch(nxt, 0, 0);
    interleave_behind_mfma<0, NMFMA, NFRAG, 0x100, 0, 0>();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 1; s < E; ++s) {
      mfma_step(1, s);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (; kt + 1 < nkt; ++kt) {
    const int cur = kt & 1, nxt = cur ^ 1;
    mfma_live(0, 0);
    lstore(nxt);
    gload(kt + 2 < nkt ? kt + 2 : nkt - 1);
    __builtin_amdgcn_sched_barrier(0);
    fetch(cur, 1, 1);
#pragma unroll
    for (int s = 1; s < E; ++s) mfma_live(0, s);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_live(1, 0);
    fetch(nxt, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 1; s < E; ++s) mfma_live(1, s);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (nkt > 0) {
    const int cur = (nkt - 1) & 1;
    fetch(cur, 1, 1);
#pragma unroll
    for (int s = 0; s < E; ++s) mfma_live(0, s);
#pragma unroll
    for (int s = 0; s < E; ++s) mfma_live(1, s);
  }

  // Epilogue.  Accumulator (j, i), register r, lane l  ->  C(row, col) with
  // row = m0 + wm0 + frag_row<GA>(i, l % 16), col = n0 + wn0 + frag_row<GB>(j, acc_row(r, l)).
  // Blocks i .. i+GA-1 hold neighbouring rows, so a lane stores them as one vector when C
  // allows it (ldc a multiple of GA on a base aligned to the vector; groups start on
  // multiples of GA).
  // A sliced tile parks its raw sums in its slot of the split workspace instead (a BM x BN
  // column-major tile: no scaling, no bounds, no triangle).
  typedef typename VecOf<T, GA>::type cvec_t;
  T alpha = p.alpha, beta = p.beta;
  T* Cp = p.C;
  long ldc = p.ldc;
  int m_lim = p.m, n_lim = p.n, tri = p.tri;
  if (sliced) {
    T* slot = p.split_ws + slot_index * (long)(BM * BN);
    Cp = slot - m0 - (long)n0 * BM;
    ldc = BM;
    alpha = T(1);
    beta = T(0);
    m_lim = m0 + BM;
    n_lim = n0 + BN;
    tri = 0;
  }
  const bool vec_ok =
      (ldc % GA == 0) && ((reinterpret_cast<uintptr_t>(Cp) & (GA * sizeof(T) - 1)) == 0);

  // Tiles that lie wholly inside C (and wholly inside the wanted triangle) on vector-aligned
  // storage: no per-element decisions.  With beta != 0 the old values of one block column
  // (4 * TM / GA vectors per lane) are all requested before the first is used; a store that
  // had to wait for its own load, one after the other, would leave the epilogue latency bound.
  const bool whole_tile = m0 + BM <= m_lim && n0 + BN <= n_lim &&
                          (tri == 0 || (tri == 1 && m0 >= n0 + BN - 1) ||
                           (tri == 2 && m0 + BM - 1 <= n0));
  if (whole_tile && vec_ok) {
    constexpr int NG = TM / GA;
    T* c0 = Cp + (m0 + wm0 + GA * r16) + (long)(n0 + wn0) * ldc;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      cvec_t old[4][NG];
      if (beta != T(0)) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int ig = 0; ig < NG; ++ig)
            old[r][ig] = *reinterpret_cast<const cvec_t*>(
                c0 + 16 * GA * ig + (long)frag_row<GB>(j, Elem<T>::acc_row(r, lane)) * ldc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int ig = 0; ig < NG; ++ig) {
          cvec_t out;
#pragma unroll
          for (int g = 0; g < GA; ++g) {
            T v = alpha * acc[j][ig * GA + g][r];
            if (beta != T(0)) v += beta * vget(old[r][ig], g);
            vset(out, g, v);
          }
          // Nontemporal: C is not read again by this launch, so it need not displace the panels
          // in L2 (65536 x 256 x 256: 129.4 -> 126.8 us; with 8-byte stores it is slower).
          __builtin_nontemporal_store(
              out, reinterpret_cast<cvec_t*>(c0 + 16 * GA * ig +
                                             (long)frag_row<GB>(j, Elem<T>::acc_row(r, lane)) * ldc));
        }
    }
    return;
  }
  if (whole_tile) {  // the same, element by element (odd ldc or unaligned C)
    T* c0 = Cp + (m0 + wm0) + (long)(n0 + wn0) * ldc;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      T old[4][TM];
      if (beta != T(0)) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int i = 0; i < TM; ++i)
            old[r][i] = c0[frag_row<GA>(i, r16) +
                           (long)frag_row<GB>(j, Elem<T>::acc_row(r, lane)) * ldc];
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          T v = alpha * acc[j][i][r];
          if (beta != T(0)) v += beta * old[r][i];
          c0[frag_row<GA>(i, r16) + (long)frag_row<GB>(j, Elem<T>::acc_row(r, lane)) * ldc] = v;
        }
    }
    return;
  }

  // Tiles that hang over the edge of C or straddle the diagonal: element by element.  The
  // old values are requested unconditionally from clamped (valid) addresses, a block column
  // at a time, so that only the stores are conditional and nothing waits on a single load.
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    T old[4][TM];
    if (beta != T(0)) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = n0 + wn0 + frag_row<GB>(j, Elem<T>::acc_row(r, lane));
        const T* ccol = Cp + (long)(col < n_lim ? col : n_lim - 1) * ldc;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int row = m0 + wm0 + frag_row<GA>(i, r16);
          old[r][i] = ccol[row < m_lim ? row : m_lim - 1];
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int col = n0 + wn0 + frag_row<GB>(j, Elem<T>::acc_row(r, lane));
      T* ccol = Cp + (long)col * ldc;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = m0 + wm0 + frag_row<GA>(i, r16);
        bool keep = col < n_lim && row < m_lim;
        if (tri == 1) keep = keep && row >= col;
        if (tri == 2) keep = keep && row <= col;
        T v = alpha * acc[j][i][r];
        if (beta != T(0)) v += beta * old[r][i];
        if (keep) ccol[row] = v;
      }
    }
  }
}

// C = beta*C on one triangle (or all) of C: the alpha == 0 / k == 0 case.
template <class T>
__global__ __launch_bounds__(256) void scale_c_kernel(int m, int n, T beta, T* C, long ldc,
                                                     int tri) {
  const int row = blockIdx.x * 256 + threadIdx.x;
  if (row >= m) return;
  for (int col = blockIdx.y; col < n; col += gridDim.y) {
    if (tri == 1 && row < col) continue;
    if (tri == 2 && row > col) continue;
    T* c = C + row + (long)col * ldc;
    *c = (beta == T(0)) ? T(0) : beta * *c;
  }
}

// Finish the sliced tiles: C(tile) = alpha * (sum of the tile's slices, in slice order) +
// beta * C(tile), with the bounds and triangle masks of the GEMM epilogue.  One workgroup per
// 8 columns of a tile.
template <class T, int BM, int BN>
__global__ __launch_bounds__(256) void reduce_kernel(GemmArgs<T> p, int whole) {
  constexpr int CB = 8;
  const int tile = blockIdx.x / (BN / CB), cb = blockIdx.x % (BN / CB);
  int tile_m, tile_n;
  tile_of_logical(whole + tile, p.tiles_m, p.tiles_n, p.tri, BM, BN, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  int slices;
  long first;
  slices_of_tile(tile, p.split_tiles, p.split_s, p.split_more, slices, first);
  const T* ws = p.split_ws + first * (long)(BM * BN);
  // Each lane owns NE elements; their loads of one slice are independent, so NE (times the
  // unroll of the slice loop) requests are in flight per lane.
  constexpr int NE = BM * CB / 256;
  T sum[NE];
#pragma unroll
  for (int q = 0; q < NE; ++q) sum[q] = T(0);
#pragma unroll 4
  for (int sl = 0; sl < slices; ++sl) {
#pragma unroll
    for (int q = 0; q < NE; ++q) {
      const int e = threadIdx.x + q * 256;
      sum[q] += ws[(long)sl * (BM * BN) + (e % BM) + (cb * CB + e / BM) * BM];
    }
  }
#pragma unroll
  for (int q = 0; q < NE; ++q) {
    const int e = threadIdx.x + q * 256;
    const int row = m0 + e % BM, col = n0 + cb * CB + e / BM;
    if (row >= p.m || col >= p.n) continue;
    if (p.tri == 1 && row < col) continue;
    if (p.tri == 2 && row > col) continue;
    T* cp = p.C + row + (long)col * p.ldc;
    T v = p.alpha * sum[q];
    if (p.beta != T(0)) v += p.beta * *cp;
    *cp = v;
  }
}

static void* split_workspace(rtat_native_handle* h) {
  return h->user_ws != nullptr ? nullptr : h->split_ws;
}
void prepare_split_workspace(rtat_native_handle* h) {
  if (h->split_ws != nullptr || h->split_ws_failed) return;
  if (malloc_on_device(h->device, &h->split_ws, SPLIT_WS_BYTES) != hipSuccess) {
    (void)hipGetLastError();
    h->split_ws = nullptr;
    h->split_ws_failed = true;
  }
}

// Macro tiles; BK is 128 bytes of k for either element type.
template <class T> using T256x128 = TileShape<256, 128, 8 * Elem<T>::E, 4, 2, 1>;  // 8 waves of 64x64
template <class T> using T128x128 = TileShape<128, 128, 8 * Elem<T>::E, 2, 2, 2>;  // 4 waves of 64x64
template <class T> using T128x64 = TileShape<128, 64, 8 * Elem<T>::E, 2, 2, 2>;    // 4 waves of 64x32
template <class T> using T64x64 = TileShape<64, 64, 8 * Elem<T>::E, 2, 2, 4>;      // 4 waves of 32x32
// For problems of a few hundred of its tiles and a short k only (pick_variant): one launch
// where the 64 x 64 shape needs K slices and a second kernel to fill the CUs.
template <class T> using T32x32 = TileShape<32, 32, 8 * Elem<T>::E, 2, 2, 4>;      // 4 waves of 16x16

template <class T, class TS, bool TA, bool TB, int VEC>
static rtat_status_t launch_tile(rtat_native_handle* h, const GemmArgs<T>& a) {
  typedef Panel<T, TA, TS::BM, TS::BK> PA;
  typedef Panel<T, !TB, TS::BN, TS::BK> PB;
  const size_t lds_bytes = 2 * (size_t)(PA::SIZE + PB::SIZE) * sizeof(T);
  auto kern = gemm_kernel<T, TS, TA, TB, VEC>;
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
  GemmArgs<T> p = a;
  // Bytes from a tile's first element to its farthest one, per operand.
  const long es = (long)sizeof(T);
  const long span_a = TA ? ((long)(TS::BM - 1) * a.lda + TS::BK) * es
                         : ((long)(TS::BK - 1) * a.lda + TS::BM) * es;
  const long span_b = !TB ? ((long)(TS::BN - 1) * a.ldb + TS::BK) * es
                          : ((long)(TS::BK - 1) * a.ldb + TS::BN) * es;
  p.wide = (span_a >= (1L << 32) || span_b >= (1L << 32)) ? 1 : 0;

  // Which tiles are computed whole, cut along K (tail splitting) or cut into 64 x 64 pieces
  // (tail subdivision): gemm_plan.h.  a.split_s carries the caller's wish, one of the SPLIT_*
  // modes of plan_launch.
  T* ws = static_cast<T*>(split_workspace(h));
  const LaunchPlan plan =
      plan_launch(a.m, a.n, a.k, a.tri, TS::BM, TS::BN, TS::BK, TS::WG_PER_CU, (int)sizeof(T),
                  h->compute_units, a.split_s, ws != nullptr, a.sub_count == 0);
  p.tiles_m = plan.tiles_m;
  p.tiles_n = plan.tiles_n;
  if (plan.tiles > 0x7fffffffL || plan.grid > 0x7fffffffL) return RTAT_STATUS_INVALID_VALUE;
  if (plan.tiles == 0) return RTAT_STATUS_SUCCESS;
  p.split_tiles = plan.split_tiles;
  p.split_s = plan.split_s;
  p.split_more = plan.split_more;
  p.split_ws = plan.split_tiles > 0 ? ws : nullptr;
  p.sub_base = p.sub_count = p.sub_bm = p.sub_bn = 0;
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  p.mask_thin = plan.tiles >= 2 * cus * TS::WG_PER_CU ? 1 : 0;
  if (a.sub_count == 0) {  // what rtat_last_launch reports
    rtat_launch_info_t& last = h->last;
    h->last_bm = TS::BM;
    h->last_bn = TS::BN;
    last.tiles = (int)plan.tiles;
    last.split_tiles = plan.split_tiles;
    last.split_slices = plan.split_tiles > 0 ? plan.split_s : 0;
    last.subdivided = (int)plan.sub_count;
  }
  if (plan.sub_count > 0) {
    // Full rounds with this shape, the leftover tiles as 64 x 64 pieces.
    hipLaunchKernelGGL(kern, dim3((unsigned)plan.lead), dim3(TS::NT), lds_bytes, h->stream, p);
    rtat_status_t st = launch_status();
    if (st != RTAT_STATUS_SUCCESS) return st;
    typedef T64x64<T> SUB;
    typedef Panel<T, TA, SUB::BM, SUB::BK> SA;
    typedef Panel<T, !TB, SUB::BN, SUB::BK> SB;
    const size_t sub_lds = 2 * (size_t)(SA::SIZE + SB::SIZE) * sizeof(T);
    static_assert(2 * (SA::SIZE + SB::SIZE) * sizeof(T) <= 65536, "no LDS attribute needed");
    static_assert(SUB::BM == 64 && SUB::BN == 64, "plan_launch counts 64 x 64 pieces");
    GemmArgs<T> q = p;
    q.sub_base = (int)plan.lead;
    q.sub_count = (int)plan.sub_count;
    q.sub_bm = TS::BM;
    q.sub_bn = TS::BN;
    q.mask_thin = 0;
    hipLaunchKernelGGL((gemm_kernel<T, SUB, TA, TB, VEC>), dim3((unsigned)plan.sub_grid),
                       dim3(SUB::NT), sub_lds, h->stream, q);
    return launch_status();
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)plan.grid), dim3(TS::NT), lds_bytes, h->stream, p);
  rtat_status_t st = launch_status();
  if (st != RTAT_STATUS_SUCCESS || plan.split_tiles == 0) return st;
  hipLaunchKernelGGL((reduce_kernel<T, TS::BM, TS::BN>), dim3((unsigned)plan.reduce_grid), dim3(256),
                     0, h->stream, p, (int)plan.whole);
  return launch_status();
}

// The panels are always fetched with 16-byte buffer loads.  A buffer load needs its address
// aligned to 4 bytes only, so an odd leading dimension or a base that is merely element-aligned
// takes the same path (measured against element-wise loads on MI355X: 65536 x 256 x 256 with
// ld = rows + 3 151.5 -> 148.5 us, 4097^3 TN 2000 -> 1975 us, nothing slower).
template <class T, class TS>
static rtat_status_t launch_ops(rtat_native_handle* h, bool ta, bool tb, const GemmArgs<T>& a) {
  constexpr int E = Elem<T>::E;
  if (!ta && !tb) return launch_tile<T, TS, false, false, E>(h, a);
  if (!ta && tb) return launch_tile<T, TS, false, true, E>(h, a);
  if (ta && !tb) return launch_tile<T, TS, true, false, E>(h, a);
  return launch_tile<T, TS, true, true, E>(h, a);
}

template <class T>
rtat_status_t launch_gemm(rtat_native_handle* h, bool ta, bool tb, int m, int n, int k, T alpha,
                          const T* A, int lda, const T* B, int ldb, T beta, T* C, int ldc,
                          int tri, int variant) {
  if (m < 0 || n < 0 || k < 0) return RTAT_STATUS_INVALID_VALUE;
  KernelOptions opt;
  if (!decode_options(variant, opt)) return RTAT_STATUS_INVALID_VALUE;
  variant = opt.tile;
  if (ldc < (m > 1 ? m : 1)) return RTAT_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0) return RTAT_STATUS_SUCCESS;
  if (C == nullptr) return RTAT_STATUS_INVALID_VALUE;
  if (alpha == T(0) || k == 0) {
    if (beta == T(1)) return RTAT_STATUS_SUCCESS;
    dim3 grid((m + 255) / 256, (unsigned)(n > 65535 ? 65535 : n));
    hipLaunchKernelGGL(scale_c_kernel<T>, grid, dim3(256), 0, h->stream, m, n, beta, C,
                       (long)ldc, tri);
    return launch_status();
  }
  const int a_rows = ta ? k : m, b_rows = tb ? n : k;
  if (A == nullptr || B == nullptr || lda < (a_rows > 1 ? a_rows : 1) ||
      ldb < (b_rows > 1 ? b_rows : 1))
    return RTAT_STATUS_INVALID_VALUE;

  GemmArgs<T> a;
  a.m = m; a.n = n; a.k = k;
  a.alpha = alpha; a.beta = beta;
  a.A = A; a.lda = lda; a.B = B; a.ldb = ldb; a.C = C; a.ldc = ldc;
  a.tiles_m = a.tiles_n = 0;
  a.tri = tri;
  a.wide = 0;
  a.split_tiles = 0;
  // The caller's tail mode as a split mode of plan_launch; under RTAT_TAIL_AUTO a fixed shape
  // takes the fixed rule and the automatic shape (below) what its heuristic priced.
  a.split_s = opt.tail == RTAT_TAIL_WHOLE   ? SPLIT_WHOLE
              : opt.tail == RTAT_TAIL_SPLIT ? SPLIT_FORCED
                                            : SPLIT_STATIC;
  a.split_more = 0;
  a.split_ws = nullptr;
  a.sub_base = a.sub_count = a.sub_bm = a.sub_bn = 0;
  a.mask_thin = 0;
  constexpr int E = Elem<T>::E;
  if (variant == RTAT_GEMM_AUTO) {
    const bool can_split = h->user_ws == nullptr && h->split_ws != nullptr;
    const Pick pick = pick_variant(h->compute_units > 0 ? h->compute_units : 256, m, n, k, 8 * E,
                                   (int)sizeof(T), tri, can_split, opt.tail);
    variant = pick.variant;
    if (opt.tail == RTAT_TAIL_AUTO) a.split_s = pick.split ? SPLIT_PRICED : SPLIT_NEVER;
  }
  switch (variant) {
    case GEMM_SHAPE_T32x32: return launch_ops<T, T32x32<T>>(h, ta, tb, a);
    case RTAT_GEMM_T256x128: return launch_ops<T, T256x128<T>>(h, ta, tb, a);
    case RTAT_GEMM_T128x128: return launch_ops<T, T128x128<T>>(h, ta, tb, a);
    case RTAT_GEMM_T128x64: return launch_ops<T, T128x64<T>>(h, ta, tb, a);
    default: return launch_ops<T, T64x64<T>>(h, ta, tb, a);
  }
}

template rtat_status_t launch_gemm<double>(rtat_native_handle*, bool, bool, int, int, int, double,
                                           const double*, int, const double*, int, double,
                                           double*, int, int, int);
template rtat_status_t launch_gemm<float>(rtat_native_handle*, bool, bool, int, int, int, float,
                                          const float*, int, const float*, int, float, float*,
                                          int, int, int);

}  // namespace rtat_native
