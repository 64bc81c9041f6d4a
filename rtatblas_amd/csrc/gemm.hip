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
//     one barrier per iteration.
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
//     guarded loads that zero-fill.  Any m, n, k, ld is accepted; odd leading dimensions or
//     unaligned bases fall back from 16-byte to element-wise loads.
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
#include "mfma.h"

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

// Row interleave of an operand with T blocks per wave: a k-major panel is read one row at a
// time, where pairs give the conflict-free lane stride; an mn-major panel is read along the
// rows, a whole vector of them when the block count allows, else a pair.
template <class T, bool KMAJOR, int TBLK>
struct RowGroup {
  static constexpr int G = KMAJOR ? 2 : (TBLK % Elem<T>::E == 0 ? Elem<T>::E : 2);
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
        for (int g = 0; g < G; ++g) f[b + g][s] = v[g];
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

// Enumerated tiles in tile rows 0 .. i-1 of a triangular C, for i < tiles_m and a tile height
// that is a multiple of the tile width: no row above the last is cut short by the edge of C,
// so row j holds (bm / bn) * (j + 1) tiles (lower) or tiles_n - (bm / bn) * j (upper).
__host__ __device__ inline long tri_rows_before(int tri, long i, int bm, int bn, int tiles_n) {
  const long r = bm / bn;
  return tri == 1 ? r * i * (i + 1) / 2 : i * tiles_n - r * i * (i - 1) / 2;
}

// Sliced tile `tile` (counted among the sliced ones): how many slices it has and the index of
// its first slice among all slices.
__host__ __device__ inline void slices_of_tile(int tile, int tiles, int s, int more, int& count,
                                               long& first) {
  const int plain = tiles - more;
  if (tile < plain) {
    count = s;
    first = (long)tile * s;
  } else {
    count = s + 1;
    first = (long)plain * s + (long)(tile - plain) * (s + 1);
  }
}

// Workgroup id -> position in the logical tile order.  Ids are dealt round-robin to the XCDs,
// so XCD x sees ids x, x+8, ...; give it one contiguous slice of the order, so that the tiles
// an XCD has in flight share A and B panels through its own L2.
__device__ inline int logical_of_workgroup(int wg, int count) {
  const int per = count / XCDS, rem = count % XCDS;
  const int x = wg % XCDS, i = wg / XCDS;
  return x * per + (x < rem ? x : rem) + i;
}

// Position in the logical tile order -> (tile row, tile column).
//   * Full C: the order walks bands of BAND tile columns, tile columns fastest across a band,
//     so the ~64 tiles an XCD has in flight share few distinct A and B panels.
//   * Triangular C: only tiles that touch the triangle are enumerated (row by row), so every
//     XCD gets the same number of real tiles.
__device__ inline void tile_of_logical(int logical, int tiles_m, int tiles_n, int tri, int bm,
                                       int bn, int& tm, int& tn) {
  if (tri != 0) {
    // The row from the root of the quadratic tri_rows_before(row) = logical, in single
    // precision, then set right by at most a step or two with the exact count.
    const float r = (float)(bm / bn), l = (float)logical;
    float est;
    if (tri == 1) {
      est = (sqrtf(1.0f + 8.0f * l / r) - 1.0f) * 0.5f;
    } else {
      const float b = (float)tiles_n + 0.5f * r, d = b * b - 2.0f * r * l;
      est = (b - sqrtf(d > 0.0f ? d : 0.0f)) / r;
    }
    int row = (int)est;
    row = row < 0 ? 0 : (row > tiles_m - 1 ? tiles_m - 1 : row);
    while (row > 0 && tri_rows_before(tri, row, bm, bn, tiles_n) > logical) --row;
    while (row + 1 < tiles_m && tri_rows_before(tri, row + 1, bm, bn, tiles_n) <= logical) ++row;
    logical -= (int)tri_rows_before(tri, row, bm, bn, tiles_n);
    tm = row;
    tn = (tri == 1) ? logical : tiles_n - tri_row_count(tri, row, bm, bn, tiles_n) + logical;
    return;
  }
  const int band_tiles = BAND * tiles_m;
  const int band = logical / band_tiles, in = logical % band_tiles;
  const int left = tiles_n - band * BAND;
  const int width = left < BAND ? left : BAND;
  tm = in / width;
  tn = band * BAND + in % width;
}

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
  // second, guarded loop.
  constexpr int NMFMA = TM * TN;
  constexpr int NMOVE = decltype(mva)::NV + decltype(mvb)::NV;  // global loads = LDS stores
  constexpr int NFRAG = (A_KMAJOR ? TM : E * TM / GA) + (B_KMAJOR ? TN : E * TN / GB);
  // When every panel is a full one the first loop also runs the last iterations, whose
  // prefetch index is clamped (the last panel is fetched again and never used).
  int kt = 0;
  const int fast_end = nkt_fast == nkt ? nkt - 1 : nkt_fast - 2;
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
    mfma_step(0, 0);
    lstore(nxt);
    gload(kt + 2 < nkt ? kt + 2 : nkt - 1);
    __builtin_amdgcn_sched_barrier(0);
    fetch(cur, 1, 1);
#pragma unroll
    for (int s = 1; s < E; ++s) mfma_step(0, s);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_step(1, 0);
    fetch(nxt, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 1; s < E; ++s) mfma_step(1, s);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (nkt > 0) {
    const int cur = (nkt - 1) & 1;
    fetch(cur, 1, 1);
#pragma unroll
    for (int s = 0; s < E; ++s) mfma_step(0, s);
#pragma unroll
    for (int s = 0; s < E; ++s) mfma_step(1, s);
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
            if (beta != T(0)) v += beta * old[r][ig][g];
            out[g] = v;
          }
          *reinterpret_cast<cvec_t*>(
              c0 + 16 * GA * ig + (long)frag_row<GB>(j, Elem<T>::acc_row(r, lane)) * ldc) = out;
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

// Device memory for the slices of the tail tiles, owned by the handle (one allocation, made
// when the handle is created).  A caller that lends its own workspace manages all device
// memory itself: then tails are not split.
constexpr size_t SPLIT_WS_BYTES = (size_t)64 << 20;
constexpr int SPLIT_MIN_KT = 8;  // K panels a slice must have to be worth a workgroup
constexpr int SPLIT_LONG_KT = 256;  // K panels from which splitting pays without a full round
constexpr int SPLIT_MID_KT = 128;   // ... or from this many when at most half the slots have a tile
constexpr int SPLIT_FEW_TILES = 8;  // ... or fewer tiles than an eighth of the workgroup slots
constexpr int SPLIT_UNEVEN_KT = 48; // ... or from this many when the tiles load the CUs unevenly

// K slices per tail tile: as many as fill the machine once more.  When the whole problem is
// smaller than one round of workgroups the second kernel only pays for a long K, or when the
// tiles are so few that most of the machine would stand idle.  1 = no split.
static long split_slices(long tiles, long slots, long nkt, bool uneven) {
  const long full = tiles / slots, tail = tiles % slots;
  if (tail == 0) return 1;
  if (full == 0 && nkt < SPLIT_LONG_KT && tiles * SPLIT_FEW_TILES > slots &&
      !(nkt >= SPLIT_MID_KT && tiles * 2 <= slots) && !uneven)
    return 1;
  long s = slots / tail;
  if (s > nkt / SPLIT_MIN_KT) s = nkt / SPLIT_MIN_KT;
  return s < 2 ? 1 : s;
}

// Which of the last tiles to cut along K, and into how many slices (tiles == 0: none); the
// last `more` of them get one slice more.
struct SplitPlan {
  long tiles, slices, more;
};
// First choice: the leftover of the last round of workgroup slots (split_slices).  When that
// leftover is too large to cut — more than half a round — the CUs still differ by one tile
// (tiles % CUs of them hold one more): cutting just those into a slice per CU (two slices each
// when they are between a third and half of the CUs) evens that out, if they are at most half
// of the CUs and every CU has a whole tile as well (with the limit at a quarter, 1600^3 took
// 143 us instead of 125 and 1856^3 217 instead of 191).
static SplitPlan split_plan(long tiles, long cus, int per_cu, long nkt, bool priced) {
  const long slots = cus * per_cu;
  // Less than a round of the smallest shape, but more tiles than CUs, and more than half of
  // the CUs hold one tile more than the rest (too many for the few-odd-tiles plan below,
  // which is the better one where it applies: 1152^3 61 -> 55 us): whole tiles would take two
  // tile times on those CUs and leave the others half idle, slices even that out (1280^3:
  // 79 -> 78 us; before the odd-tiles plan reached up to half the CUs this rule served from a
  // quarter on: 1152^3 71 -> 61 us, DSYRK 1600/1600 100 -> 81).
  const bool uneven = per_cu >= 4 && tiles > cus && tiles < slots && (tiles % cus) * 2 > cus &&
                      nkt >= SPLIT_UNEVEN_KT;
  // At most one tile of the smallest shape per CU: whether slices pay depends on k and on how
  // many CUs the tiles leave idle, which the shape heuristic prices; a caller that has priced
  // the split (`priced`) may have it (832^3: 29.1 -> 27.1 us, DSYRK 1024/1024: 37.7 -> 32.6,
  // DSYRK 1088/1088: 40.0 -> 33.6), a fixed shape keeps the rule (64 x 64 at 1024^3 would go
  // from 36.2 to 41.8 us).
  const bool sparse = priced && per_cu >= 4 && tiles <= cus;
  long s = split_slices(tiles, slots, nkt, uneven || sparse);
  // A small leftover behind full rounds (at most a quarter of the CUs): one slice per CU
  // rather than one per slot.  Each then has its CU to itself, and half as many partial tiles
  // go through scratch (n = 3072: 823 -> 782 us; DSYRK 8192/2048: 1911 -> 1888 us).
  if (s >= 2 && tiles >= slots && per_cu > 1 && (tiles % slots) * 4 <= cus) {
    const long one_per_cu = cus / (tiles % slots);
    if (one_per_cu >= 2 && one_per_cu < s) s = one_per_cu;
  }
  // The same for a problem of less than one round, where the slices then still occupy at
  // least 85 % of the CUs (512x512x8192: 78 -> 70 us, 1024x1024x4000: 141 -> 126 us,
  // 128x128x65536: 68 -> 46 us); otherwise every slot gets a slice (below).
  // A lone workgroup of the smallest shape does not keep a CU busy unless its slice is short
  // (four or more per tile): otherwise that shape gets two slices per CU.
  if (s >= 2 && tiles < slots && per_cu > 1) {
    const long wanted = (per_cu >= 4 && cus / tiles < 4) ? 2 * cus : cus;
    long fewer = wanted / tiles;
    if (fewer > nkt / SPLIT_MIN_KT) fewer = nkt / SPLIT_MIN_KT;
    if (fewer >= 2 && fewer < s && tiles * fewer * 100 >= wanted * 85) return {tiles, fewer, 0};
  }
  if (s >= 2) {
    // When the slices are all there is to run (less than a round of tiles), the slots they
    // leave empty are filled by giving that many tiles one slice more; a CU then holds a mix
    // of longer and shorter slices.  Not with one workgroup per CU, where the longest slice
    // would still set the pace, and not behind full rounds of whole tiles, whose slots free
    // up one by one anyway (measured: up to 2 % slower there).
    const long tail = tiles % slots;
    long more = slots - tail * s;
    if (tiles >= slots || per_cu < 2 || s + 1 > nkt / SPLIT_MIN_KT || more >= tail) more = 0;
    return {tail, s, more};
  }
  const long odd = tiles % cus;
  if (per_cu > 1 && odd != 0 && odd * 2 <= cus && tiles > cus) {
    long so = cus / odd;
    if (so > nkt / SPLIT_MIN_KT) so = nkt / SPLIT_MIN_KT;
    if (so >= 2) return {odd, so, 0};
  }
  return {0, 1, 0};
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

// Tail subdivision: when the tiles left over after the last full round are too many to be
// cut along K (less than two slices each would fit) but fewer than fill the machine, CUs
// with two leftover tiles set the pace while others hold one or none.  Cut into 64 x 64
// pieces by a second launch, the same work spreads evenly over the CUs.  Worth it when the
// leftover is more than one tile per CU and less than what the smaller shape's lower rate
// gives back.
// Measured rate of the subdivided phase (64 x 64 pieces, a second launch behind the first)
// relative to full rounds of the larger shape: 0.66 .. 0.8 at n = 2560, 3584 and 3840 on MI355X.
constexpr double SUB_RATE = 0.72;
static bool subdivide_tail(int bm, int bn, int per_cu, long tail, long cus) {
  if (bm == 64 && bn == 64) return false;
  const long slots = cus * per_cu;
  // With at most one leftover workgroup per CU (half a CU's worth for a one-per-CU shape)
  // each runs alone on its CU and is nearly twice as fast: nothing to gain.
  const long least = per_cu > 1 ? cus : cus / 2;
  return tail > least && (double)tail < (SUB_RATE - 0.02) * (double)slots;
}

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
  p.tiles_m = (a.m + TS::BM - 1) / TS::BM;
  p.tiles_n = (a.n + TS::BN - 1) / TS::BN;
  long tiles = (long)p.tiles_m * p.tiles_n;
  if (a.tri != 0) {
    tiles = 0;
    for (int i = 0; i < p.tiles_m; ++i) tiles += tri_row_count(a.tri, i, TS::BM, TS::BN, p.tiles_n);
  }
  if (tiles > 0x7fffffffL) return RTAT_STATUS_INVALID_VALUE;
  if (tiles == 0) return RTAT_STATUS_SUCCESS;

  // Tail splitting.  The CUs hold `slots` workgroups at a time; the tiles % slots tiles left
  // after the last full round would occupy part of the machine for a whole tile time.  Cut
  // them into as many K slices as fill the machine once more, each at least SPLIT_MIN_KT panels.
  p.split_tiles = 0;
  p.split_s = 1;
  p.split_more = 0;
  p.split_ws = nullptr;
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  const long slots = cus * TS::WG_PER_CU;
  const long tail = tiles % slots;
  const int nkt = (a.k + TS::BK - 1) / TS::BK;
  if (tail > 0 && a.split_s != 0) {
    const SplitPlan plan = split_plan(tiles, cus, TS::WG_PER_CU, nkt, a.split_s == 2);
    long s_want = plan.slices, more = plan.more;
    if (plan.tiles > 0) {  // the slices the scratch has room for
      const long room = (long)(SPLIT_WS_BYTES / ((size_t)TS::BM * TS::BN * sizeof(T)));
      if (plan.tiles * s_want + more > room) {
        more = 0;
        if (s_want > room / plan.tiles) s_want = room / plan.tiles;
      }
    }
    if (s_want >= 2 && s_want + (more > 0 ? 1 : 0) <= nkt) {  // no slice without a panel
      T* ws = static_cast<T*>(split_workspace(h));
      if (ws != nullptr) {
        p.split_tiles = (int)plan.tiles;
        p.split_s = (int)s_want;
        p.split_more = (int)more;
        p.split_ws = ws;
      }
    }
  }
  p.sub_base = p.sub_count = p.sub_bm = p.sub_bn = 0;
  if (p.split_tiles == 0 && tiles >= slots && a.sub_count == 0 &&
      subdivide_tail(TS::BM, TS::BN, TS::WG_PER_CU, tail, cus)) {
    // Full rounds with this shape, the leftover tiles as 64 x 64 pieces.
    const long lead = tiles - tail;
    hipLaunchKernelGGL(kern, dim3((unsigned)lead), dim3(TS::NT), lds_bytes, h->stream, p);
    rtat_status_t st = launch_status();
    if (st != RTAT_STATUS_SUCCESS) return st;
    typedef T64x64<T> SUB;
    typedef Panel<T, TA, SUB::BM, SUB::BK> SA;
    typedef Panel<T, !TB, SUB::BN, SUB::BK> SB;
    const size_t sub_lds = 2 * (size_t)(SA::SIZE + SB::SIZE) * sizeof(T);
    static_assert(2 * (SA::SIZE + SB::SIZE) * sizeof(T) <= 65536, "no LDS attribute needed");
    GemmArgs<T> q = p;
    q.sub_base = (int)lead;
    q.sub_count = (int)tail;
    q.sub_bm = TS::BM;
    q.sub_bn = TS::BN;
    const long pieces = (TS::BM / SUB::BM) * (TS::BN / SUB::BN);
    const long groups = (tail + XCDS - 1) / XCDS;
    hipLaunchKernelGGL((gemm_kernel<T, SUB, TA, TB, VEC>), dim3((unsigned)(groups * pieces * XCDS)),
                       dim3(SUB::NT), sub_lds, h->stream, q);
    return launch_status();
  }
  const long whole = tiles - p.split_tiles;
  const long nwg = whole + (long)p.split_tiles * p.split_s + p.split_more;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(TS::NT), lds_bytes, h->stream, p);
  rtat_status_t st = launch_status();
  if (st != RTAT_STATUS_SUCCESS || p.split_tiles == 0) return st;
  hipLaunchKernelGGL((reduce_kernel<T, TS::BM, TS::BN>), dim3((unsigned)(p.split_tiles * (TS::BN / 8))),
                     dim3(256), 0, h->stream, p, (int)whole);
  return launch_status();
}

template <class T, class TS>
static rtat_status_t launch_ops(rtat_native_handle* h, bool ta, bool tb, bool vec,
                                const GemmArgs<T>& a) {
  constexpr int E = Elem<T>::E;
  if (vec) {
    if (!ta && !tb) return launch_tile<T, TS, false, false, E>(h, a);
    if (!ta && tb) return launch_tile<T, TS, false, true, E>(h, a);
    if (ta && !tb) return launch_tile<T, TS, true, false, E>(h, a);
    return launch_tile<T, TS, true, true, E>(h, a);
  }
  if (!ta && !tb) return launch_tile<T, TS, false, false, 1>(h, a);
  if (!ta && tb) return launch_tile<T, TS, false, true, 1>(h, a);
  if (ta && !tb) return launch_tile<T, TS, true, false, 1>(h, a);
  return launch_tile<T, TS, true, true, 1>(h, a);
}

// Shape heuristic for RTAT_GEMM_AUTO.  A CU runs `per_cu` workgroups of a shape at a time;
// a launch lasts (rounds of tiles per CU) x (tile area) x (k / rate + fixed), where rate is
// the shape's measured steady-state rate relative to 128x128 and `fixed` the prologue and
// epilogue of a tile in units of k.  With tail splitting the last partial round costs only
// its share (plus the small reduction pass); without it (short k) it costs a whole round,
// somewhat less when its workgroups have their CUs to themselves.  A CU that only ever holds
// one workgroup has nothing to run while that one sits in its barrier, prologue or epilogue.
// Constants fitted on MI355X (n = 1024 .. 16384, k up to 32768).
struct Pick {
  int variant;
  bool split;  // whether the leftover tiles are to be cut along K (where the rule allows it)
};

static Pick pick_variant(const rtat_native_handle* h, int m, int n, int k, int bk, int es, int tri,
                         bool can_split) {
  const long cus = h->compute_units > 0 ? h->compute_units : 256;
  struct Cand { int id, bm, bn, per_cu; double rate; };
  const Cand cands[] = {{RTAT_GEMM_T128x128, 128, 128, 2, 1.0},
                        {RTAT_GEMM_T256x128, 256, 128, 1, 0.99},
                        {RTAT_GEMM_T128x64, 128, 64, 2, 0.96},
                        {RTAT_GEMM_T64x64, 64, 64, 4, 0.93}};
  const long nkt = (k + bk - 1) / bk;
  // A k of at most eight panels leaves a tile little more than its C traffic to do: the launch
  // is bound by memory latency, and the smallest shape, with four workgroups per CU to hide
  // it, measured 5-20 % faster than the larger ones (n = 2048 .. 12000, k = 16 .. 128).
  if (nkt <= 8 && (long)((m + 63) / 64) * ((n + 63) / 64) >= (tri == 0 ? 4 : 8) * cus)
    return {RTAT_GEMM_T64x64, true};
  Pick best = {RTAT_GEMM_T128x128, true};
  double best_cost = 0.0;
  for (const Cand& c : cands) {
    const int tm = (m + c.bm - 1) / c.bm, tn = (n + c.bn - 1) / c.bn;
    long tiles = (long)tm * tn;
    if (tri != 0) {
      tiles = 0;
      for (int i = 0; i < tm; ++i) tiles += tri_row_count(tri, i, c.bm, c.bn, tn);
    }
    const long slots = cus * c.per_cu;
    const long full = tiles / slots, tail = tiles % slots;
    const double area = (double)c.per_cu * c.bm * c.bn;
    // One round = per_cu tiles on every CU.  The leftover tiles either as they are (cut into
    // pieces where that applies) ...
    double rounds = (double)full;
    bool lone = false;
    if (tail > 0) {
      if (full >= 1 && subdivide_tail(c.bm, c.bn, c.per_cu, tail, cus)) {
        rounds += (double)tail / (double)slots * c.rate / SUB_RATE + 0.03;
      } else {
        const long per_cu_tail = (tail + cus - 1) / cus;  // workgroups a CU holds in the tail
        rounds += (double)per_cu_tail / (double)c.per_cu * (per_cu_tail < c.per_cu ? 1.15 : 1.0);
        lone = full == 0 && per_cu_tail < 2 && c.per_cu > 1;
      }
    }
    double cost =
        rounds * area * ((double)k / (c.rate * (lone ? 0.975 : 1.0)) + (lone ? 400.0 : 230.0));
    bool split = false;
    // ... or cut along K, where the rule allows it: a fraction of a round, plus the slices'
    // trip through scratch (written and read back once at about 4 TB/s) and a second launch
    // of some 4 us; a CU retires 512 / es products per cycle at 2.4 GHz.
    if (tail > 0 && can_split) {
      const SplitPlan plan = split_plan(tiles, cus, c.per_cu, nkt, true);
      long slices = plan.slices, more = plan.more;
      if (plan.tiles > 0) {
        const long room = (long)(SPLIT_WS_BYTES / ((size_t)c.bm * c.bn * es));
        if (plan.tiles * slices + more > room) {
          more = 0;
          if (slices > room / plan.tiles) slices = room / plan.tiles;
        }
      }
      if (slices >= 2) {
        const long slice_wgs = plan.tiles * slices + more;
        const double bytes = 2.0 * (double)slice_wgs * c.bm * c.bn * es;
        const double trip = (4e-6 + bytes / 4e12) * 2.4e9 * (512.0 / es);
        // Whole tiles: full rounds, then whatever every CU still holds (fewer than per_cu
        // workgroups share a CU somewhat less efficiently), then the slices.
        const long whole = tiles - plan.tiles;
        const long held = (whole % slots) / cus;  // plan.tiles == tiles % slots: 0
        const double thin =  // 1.15 with a single workgroup on a CU, 1.0 with all per_cu
            held > 0 && c.per_cu > 1
                ? 1.0 + 0.15 * (double)(c.per_cu - held) / (double)(c.per_cu - 1)
                : 1.0;
        const double whole_rounds =
            (double)(whole / slots) + (double)held / (double)c.per_cu * thin;
        // The slices last at least one slice's time — a round's time over the slice count
        // when they fill every workgroup slot, less when a CU holds fewer of them — and
        // longer when they outnumber the slots.
        long on_cu = (slice_wgs + cus - 1) / cus;
        if (on_cu > c.per_cu) on_cu = c.per_cu;
        double one_slice = (double)on_cu / (double)c.per_cu * (on_cu < c.per_cu ? 1.15 : 1.0) /
                           (double)slices;
        if (more > 0) {
          // Every slot holds a slice; a CU has `longer` of the longer ones (the tiles with
          // fewer slices come first and spread over the CUs) and shorter ones beside them.
          long longer = ((plan.tiles - more) * slices + cus - 1) / cus;
          if (longer > c.per_cu) longer = c.per_cu;
          one_slice = ((double)longer / (double)slices +
                       (double)(c.per_cu - longer) / (double)(slices + 1)) / (double)c.per_cu;
        }
        const double by_count = (double)plan.tiles / (double)slots;
        const double sliced = (one_slice > by_count ? one_slice : by_count) + 0.02;
        const double cut = (whole_rounds + sliced) * area * ((double)k / c.rate + 230.0) + trip;
        if (cut < cost) {
          cost = cut;
          split = true;
        }
      }
    }
    if (best_cost == 0.0 || cost < best_cost) {
      best_cost = cost;
      best = {c.id, split};
    }
  }
  return best;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <class T>
rtat_status_t launch_gemm(rtat_native_handle* h, bool ta, bool tb, int m, int n, int k, T alpha,
                          const T* A, int lda, const T* B, int ldb, T beta, T* C, int ldc,
                          int tri, int variant) {
  if (m < 0 || n < 0 || k < 0) return RTAT_STATUS_INVALID_VALUE;
  if (variant < 0 || variant >= RTAT_GEMM_VARIANT_COUNT) return RTAT_STATUS_INVALID_VALUE;
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
  a.split_s = 1;  // 0 would forbid tail splitting, 2 says that the shape heuristic priced it
  a.split_more = 0;
  a.split_ws = nullptr;
  a.sub_base = a.sub_count = a.sub_bm = a.sub_bn = 0;
  // 16-byte vector loads need leading dimensions that are whole vectors on 16-byte aligned bases.
  constexpr int E = Elem<T>::E;
  const bool vec = aligned16(A) && aligned16(B) && (lda % E == 0) && (ldb % E == 0);
  if (variant == RTAT_GEMM_AUTO) {
    const bool can_split = h->user_ws == nullptr && h->split_ws != nullptr;
    const Pick pick = pick_variant(h, m, n, k, 8 * E, (int)sizeof(T), tri, can_split);
    variant = pick.variant;
    a.split_s = pick.split ? 2 : 0;  // 2: the split has been priced
  }
  switch (variant) {
    case RTAT_GEMM_T256x128: return launch_ops<T, T256x128<T>>(h, ta, tb, vec, a);
    case RTAT_GEMM_T128x128: return launch_ops<T, T128x128<T>>(h, ta, tb, vec, a);
    case RTAT_GEMM_T128x64: return launch_ops<T, T128x64<T>>(h, ta, tb, vec, a);
    default: return launch_ops<T, T64x64<T>>(h, ta, tb, vec, a);
  }
}

template rtat_status_t launch_gemm<double>(rtat_native_handle*, bool, bool, int, int, int, double,
                                           const double*, int, const double*, int, double,
                                           double*, int, int, int);
template rtat_status_t launch_gemm<float>(rtat_native_handle*, bool, bool, int, int, int, float,
                                          const float*, int, const float*, int, float, float*,
                                          int, int, int);

}  // namespace rtat_native
