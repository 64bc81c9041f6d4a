// Launch planning of the GEMM / SYRK core: which tiles a launch computes whole, which it
// cuts along K or into smaller pieces, how workgroup ids map to tiles, and which tile shape
// RTAT_GEMM_AUTO picks.  Pure integer / floating-point arithmetic with no device state, kept
// apart from the kernels so that it also compiles for the host alone: the same functions
// drive the launcher (gemm.hip), run inside the kernel (the id -> tile maps) and are swept by
// a CPU test over shapes, CU counts and scratch sizes for the invariants the kernel's
// addressing relies on (tests/cpp).
#pragma once
#include <math.h>
#include <stddef.h>

#include "rtat_native.h"

#if defined(__HIPCC__)
#define RTAT_HD __host__ __device__
#else
#define RTAT_HD
#endif

namespace rtat_native {

constexpr int XCDS = 8;
// A tile shape that only the automatic choice uses (32 x 32, four waves of 16 x 16): it has no
// id in rtat_gemm_variant_t, so no caller can ask for it by number.
constexpr int GEMM_SHAPE_T32x32 = RTAT_GEMM_VARIANT_COUNT;
constexpr int BAND = 4;  // tile columns per band of the tile walk
constexpr int TRI_SUPER = 8;  // tiles per side of a super-block of the walk over a triangular C

// Tiles of a triangular C (SYRK) that hold at least one element of the wanted triangle, per
// tile row i: lower (tri == 1) keeps columns [0, count), upper (tri == 2) keeps
// [tiles_n - count, tiles_n).  Shared by the launcher (grid size) and the kernel (mapping).
RTAT_HD inline int tri_row_count(int tri, int i, int bm, int bn, int tiles_n) {
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
RTAT_HD inline long tri_rows_before(int tri, long i, int bm, int bn, int tiles_n) {
  const long r = bm / bn;
  return tri == 1 ? r * i * (i + 1) / 2 : i * tiles_n - r * i * (i - 1) / 2;
}

// Sliced tile `tile` (counted among the sliced ones): how many slices it has and the index of
// its first slice among all slices.
RTAT_HD inline void slices_of_tile(int tile, int tiles, int s, int more, int& count,
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
RTAT_HD inline int logical_of_workgroup(int wg, int count) {
  const int per = count / XCDS, rem = count % XCDS;
  const int x = wg % XCDS, i = wg / XCDS;
  return x * per + (x < rem ? x : rem) + i;
}

// Position in the logical tile order -> (tile row, tile column).
//   * Full C: the order walks bands of BAND tile columns, tile columns fastest across a band,
//     so the ~64 tiles an XCD has in flight share few distinct A and B panels.
//   * Triangular C: only tiles that touch the triangle are enumerated, so every XCD gets the
//     same number of real tiles: in super-blocks for square tiles, row by row otherwise.
RTAT_HD inline void tile_of_logical(int logical, int tiles_m, int tiles_n, int tri, int bm,
                                       int bn, int& tm, int& tn) {
  if (tri != 0 && bm == bn) {
    // Square tiles: the triangle is walked in super-blocks of TRI_SUPER x TRI_SUPER tiles, the
    // super-blocks row by row and the tiles inside one row by row (the lower triangle; the
    // upper one is its mirror image).  The ~64 tiles an XCD has in flight then share 16 row
    // panels of A instead of 65 (a whole tile row shares one panel and needs 64 others).
    const int S = TRI_SUPER, T = tiles_m;
    // Tile row of the plain row-by-row count that holds `logical`: the super-row follows from
    // it, because the tiles in front of super-row I are a triangle of S I tile rows.
    const float l = (float)logical;
    int row = (int)((sqrtf(1.0f + 8.0f * l) - 1.0f) * 0.5f);
    row = row < 0 ? 0 : (row > T - 1 ? T - 1 : row);
    while (row > 0 && (long)row * (row + 1) / 2 > logical) --row;
    while (row + 1 < T && (long)(row + 1) * (row + 2) / 2 <= logical) ++row;
    const int base = row / S * S;                 // first tile row of the super-row
    const int h = T - base < S ? T - base : S;    // its height (the last one may be short)
    int rem = logical - (int)((long)base * (base + 1) / 2);
    const int full = base * h;                    // tiles of the full super-blocks left of the diagonal one
    int a, b;
    if (rem < full) {
      const int blk = rem / (h * S), in = rem % (h * S);
      a = base + in / S;
      b = blk * S + in % S;
    } else {
      rem -= full;
      int r = 0;
      while ((r + 1) * (r + 2) / 2 <= rem) ++r;
      a = base + r;
      b = base + rem - r * (r + 1) / 2;
    }
    tm = tri == 1 ? a : b;
    tn = tri == 1 ? b : a;
    return;
  }
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


// ---- tail splitting ---------------------------------------------------------------------------
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
inline long split_slices(long tiles, long slots, long nkt, bool uneven) {
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
// mode: SPLIT_STATIC the fixed rule, SPLIT_PRICED the caller has priced the split with the shape
// heuristic, SPLIT_FORCED the caller wants a split wherever two slices or more fit.  es: bytes of
// an element.
constexpr int SPLIT_NEVER = 0, SPLIT_STATIC = 1, SPLIT_PRICED = 2, SPLIT_FORCED = 3,
              SPLIT_WHOLE = 4;  // SPLIT_WHOLE: neither slices nor subdivision (plan_launch)
inline SplitPlan split_plan(long tiles, long cus, int per_cu, long nkt, int mode, int es = 8) {
  const bool priced = mode == SPLIT_PRICED || mode == SPLIT_FORCED;
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
  long s = split_slices(tiles, slots, nkt, uneven || sparse || mode == SPLIT_FORCED);
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
    // For the smallest shape three quarters of those suffice when that leaves three slices or
    // more of a middling k (40 to 64 panels): the alternative there is six or seven short
    // slices per tile, or none (768^3: 27.3 us whole, 29.0 in six slices, 25.6 in three;
    // 768 x 704 x 768 28.4 -> 24.8, 530 x 1000 x 768 29.7 -> 26.3, 704 x 832 x 1024 31.9 -> 30.0, DSYRK
    // 1024/1024 33.0 -> 31.7).  Below that k whole tiles are ahead (k = 512: 19.5 against 22.9
    // us), above it the many slices (768 x 704 x 1536: 37.3 against 39.2), and two slices a tile
    // lose to five at every k (960 x 832 x 2048: 61.0 against 66.7).  In single precision, whose
    // slices cost half as much to move, the window closes a little earlier (768^3-sized tiles:
    // k = 1536, 48 panels, 27.0 -> 24.3 us; k = 2048, 64 panels, 28.7 -> 29.3).
    const long enough =
        (per_cu >= 4 && fewer >= 3 && nkt >= 40 && nkt <= (es >= 8 ? 64 : 56)) ? 75 : 85;
    if (fewer >= 2 && fewer < s && tiles * fewer * 100 >= wanted * enough) return {tiles, fewer, 0};
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
  // Not below 20 panels: two slices of eight panels each cost more than they even out
  // (896 x 1536 x 256: 20.9 us against 19.8 whole, 1024 x 1280 x 256 20.3 / 19.8, DSYRK 1536/256 22.1 /
  // 21.2; level at k = 320, ahead from 384 on: 24.8 against 27.1).
  const long odd = tiles % cus;
  if (per_cu > 1 && odd != 0 && odd * 2 <= cus && tiles > cus && nkt >= 20) {
    long so = cus / odd;
    if (so > nkt / SPLIT_MIN_KT) so = nkt / SPLIT_MIN_KT;
    if (so >= 2) return {odd, so, 0};
  }
  return {0, 1, 0};
}

// Slices of BM x BN elements of `es` bytes the split scratch holds.
inline long split_room(int bm, int bn, int es) {
  return (long)(SPLIT_WS_BYTES / ((size_t)bm * (size_t)bn * (size_t)es));
}
// Fit a plan of `tiles` tiles x `slices` slices (+ `more` extra slices) into `room` slots:
// drop the extra slices first, then lower the slice count.  One rule for the launcher and
// for the shape heuristic that prices the split.
inline void clamp_to_room(long tiles, long& slices, long& more, long room) {
  if (tiles <= 0) return;
  if (tiles * slices + more > room) {
    more = 0;
    if (slices > room / tiles) slices = room / tiles;
  }
}

// Tail subdivision: when the tiles left over after the last full round are too many to be
// cut along K (less than two slices each would fit) but fewer than fill the machine, CUs
// with two leftover tiles set the pace while others hold one or none.  Cut into 64 x 64
// pieces by a second launch, the same work spreads evenly over the CUs.  Worth it when the
// leftover is more than one tile per CU and less than what the smaller shape's lower rate
// gives back.
// Measured rate of the subdivided phase (64 x 64 pieces, a second launch behind the first)
// relative to full rounds of the larger shape: 0.66 .. 0.8 at n = 2560, 3584 and 3840 on MI355X.
constexpr double SUB_RATE = 0.72;
inline bool subdivide_tail(int bm, int bn, int per_cu, long tail, long cus) {
  if (bm <= 64 && bn <= 64) return false;
  const long slots = cus * per_cu;
  // With at most one leftover workgroup per CU (half a CU's worth for a one-per-CU shape)
  // each runs alone on its CU and is nearly twice as fast: nothing to gain.
  const long least = per_cu > 1 ? cus : cus / 2;
  return tail > least && (double)tail < (SUB_RATE - 0.02) * (double)slots;
}


// ---- one launch, planned ------------------------------------------------------------------------
// What launch_tile enqueues for an m x n x k problem on tiles of bm x bn x bk: either
//   * one launch of `grid` workgroups: `whole` tiles computed whole (ids remapped per XCD by
//     logical_of_workgroup), then split_tiles tiles cut along K into split_s slices each, the
//     last split_more of them into one more, followed by a reduce launch; or
//   * (sub_count > 0) `lead` whole tiles of this shape, then the last sub_count tiles as
//     64 x 64 pieces by a second launch of sub_grid workgroups.
struct LaunchPlan {
  int tiles_m, tiles_n;
  long tiles;                       // enumerated tiles (those touching the wanted triangle)
  long whole, grid;                 // first launch
  int split_tiles, split_s, split_more;
  long reduce_grid;                 // workgroups of the reduce launch (0: none)
  long lead, sub_count, sub_grid;   // subdivision (sub_count == 0: none)
};

// split_mode: SPLIT_NEVER no slices (the leftover may still be subdivided), SPLIT_STATIC the
// fixed rule, SPLIT_PRICED the shape heuristic has priced the split, SPLIT_FORCED slices
// wherever two or more fit, SPLIT_WHOLE every tile whole (no slices, no subdivision).
// have_scratch: the slices have somewhere to go.  allow_sub: the leftover may be subdivided
// (false for the subdivision launch itself).
inline LaunchPlan plan_launch(int m, int n, int k, int tri, int bm, int bn, int bk, int per_cu,
                              int es, long cus, int split_mode, bool have_scratch, bool allow_sub) {
  LaunchPlan p = {};
  p.tiles_m = (m + bm - 1) / bm;
  p.tiles_n = (n + bn - 1) / bn;
  p.tiles = (long)p.tiles_m * p.tiles_n;
  if (tri != 0) {
    p.tiles = 0;
    for (int i = 0; i < p.tiles_m; ++i) p.tiles += tri_row_count(tri, i, bm, bn, p.tiles_n);
  }
  p.split_s = 1;
  if (p.tiles == 0) return p;
  if (cus <= 0) cus = 256;
  const long slots = cus * per_cu, tail = p.tiles % slots;
  const long nkt = (k + bk - 1) / bk;
  // Tail splitting.  The CUs hold `slots` workgroups at a time; the tiles % slots tiles left
  // after the last full round would occupy part of the machine for a whole tile time.
  if (split_mode == SPLIT_WHOLE) allow_sub = false;
  if (tail > 0 && split_mode != SPLIT_NEVER && split_mode != SPLIT_WHOLE && have_scratch) {
    const SplitPlan plan = split_plan(p.tiles, cus, per_cu, nkt, split_mode, es);
    long s_want = plan.slices, more = plan.more;
    clamp_to_room(plan.tiles, s_want, more, split_room(bm, bn, es));
    if (plan.tiles > 0 && s_want >= 2 && s_want + (more > 0 ? 1 : 0) <= nkt) {  // no slice without a panel
      p.split_tiles = (int)plan.tiles;
      p.split_s = (int)s_want;
      p.split_more = (int)more;
    }
  }
  if (p.split_tiles == 0 && p.tiles >= slots && allow_sub && subdivide_tail(bm, bn, per_cu, tail, cus)) {
    p.lead = p.tiles - tail;
    p.sub_count = tail;
    const long pieces = (long)(bm / 64) * (bn / 64);
    p.sub_grid = (tail + XCDS - 1) / XCDS * pieces * XCDS;
    p.whole = p.lead;
    p.grid = p.lead;
    return p;
  }
  p.whole = p.tiles - p.split_tiles;
  p.grid = p.whole + (long)p.split_tiles * p.split_s + p.split_more;
  p.reduce_grid = (long)p.split_tiles * (bn / 8);
  return p;
}

// K panels [first, first + count) of slice `slice` of `slices` over `panels` panels, as the
// kernel cuts them (the last slice also takes a ragged last panel).
RTAT_HD inline void slice_panels(long panels, int slices, int slice, long& first, long& count) {
  first = slice * panels / slices;
  count = (slice + 1) * panels / slices - first;
}

// ---- shape heuristic ----------------------------------------------------------------------------
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

// tail: the caller's rtat_tail_mode_t.  RTAT_TAIL_WHOLE prices every shape with its leftover
// tiles whole (neither slices nor subdivision), RTAT_TAIL_SPLIT takes the sliced form of every
// shape that has one.
inline Pick pick_variant(long cus, int m, int n, int k, int bk, int es, int tri, bool can_split,
                         int tail_mode = RTAT_TAIL_AUTO) {
  if (tail_mode == RTAT_TAIL_WHOLE) can_split = false;
  // Relative rates of the shapes in full rounds.  A triangular C has its own: there the
  // smallest shape loses less to the larger ones (half the waste on the diagonal tiles; it and
  // the 128 x 128 shape walk the triangle in super-blocks, which the 128 x 64 shape does not) and
  // the 256 x 128 shape is never near the front.  Over 78 DSYRK problems (n = 1536 ... 8192, 3000,
  // 5000, 7000; k = 128 ... 4096) the 64 x 64 shape was the fastest or within 1 % of it up to
  // n = 6144 and within 2.6 % beyond; with the rates of a full C the choice was 1.6 % behind the
  // best forced shape on average and more than 3 % behind in 17 of the 78 (16 % at worst), with
  // these 0.9 % and 9 (0.985 for the 64 x 64 shape, which the same table suggests, took n = 7168
  // and 8192 away from the 128 x 128 shape at a loss of 4-7 %).
  // (Measured in double precision only: single precision keeps one set of rates.)
  const bool dtri = tri != 0 && es == 8;
  struct Cand { int id, bm, bn, per_cu; double rate; };
  const Cand cands[] = {{RTAT_GEMM_T128x128, 128, 128, 2, 1.0},
                        {RTAT_GEMM_T256x128, 256, 128, 1, dtri ? 0.90 : 0.99},
                        {RTAT_GEMM_T128x64, 128, 64, 2, dtri ? 0.95 : 0.96},
                        {RTAT_GEMM_T64x64, 64, 64, 4, dtri ? 0.96 : 0.93}};
  const long nkt = (k + bk - 1) / bk;
  // Small problems: up to two 32 x 32 tiles per CU and a k of at most 32 panels (48 from one
  // tile per CU on).  The 64 x 64 shape has too few tiles there to fill the CUs and gets there
  // with K slices and the kernel that sums them, two launches of 10-15 us together; 32 x 32
  // tiles fill the machine in one, whose K loop is the shorter chain up to that k.  Measured on
  // MI355X, NN, old -> new: 512^3 14.4 -> 11.0 us (hipBLAS 11.9), 256^3 10.1 -> 6.6 (17.1),
  // 384^3 11.9 -> 9.0 (14.7), 200 x 300 x 400 12.5 -> 9.7 (10.3), 100^3 8.6 -> 5.0 (9.5),
  // 2048 x 32 x 256 12.1 -> 6.9, 640^3 20.0 -> 18.8; beyond (768^3, 512 x 512 x 1024, ...) the
  // sliced form stays ahead.
  {
    const long tm32 = (m + 31) / 32, tn32 = (n + 31) / 32;
    const long tiles32 = tri == 0 ? tm32 * tn32 : tm32 * (tm32 + 1) / 2;  // a triangle: m == n
    // A triangle (SYRK) gains as much up to 16 panels and from four tiles per five CUs on up
    // to 32 (n = 512, k = 256: 12.5 -> 8.3 us, n = 768, k = 512: 20.6 -> 17.7); with fewer tiles
    // and that k its N form, whose panels both run along m, is level or behind.
    const bool fits = tri == 0 ? (nkt <= 32 || (nkt <= 48 && tiles32 >= cus))
                               : (nkt <= 16 || (nkt <= 32 && tiles32 * 5 >= cus * 4));
    if (tiles32 * 10 <= cus * 19 && fits && tail_mode != RTAT_TAIL_SPLIT)
      return {GEMM_SHAPE_T32x32, false};
  }
  // A k of at most eight panels leaves a tile little more than its C traffic to do: the launch
  // is bound by memory latency, and the smallest shape, with four workgroups per CU to hide
  // it, measured 5-25 % faster than the larger ones up to some 48 of its tiles per CU
  // (n = 2048 .. 7000, 8192 x 2048, k = 16 .. 128; in double precision the fit above decides
  // from the second panel on, this rule serves a single panel, single precision and a
  // triangular C).  Beyond that the larger shapes, with a
  // quarter of the workgroups to dispatch, are level or ahead again (8192^2, 16384 x 4096 and
  // 12000^2 with k = 32 .. 128: 128 x 128 up to 10 % faster) and the model below chooses;
  // a single panel (k <= 16 doubles) stays with the smallest shape at every size.
  const long tiles64 = (long)((m + 63) / 64) * ((n + 63) / 64);
  // Double precision, a full C, two to ten panels: which shape is ahead there depends on how
  // the tiles of each divide among the CUs more than on anything else (3072^2, 2304 tiles of
  // 64 x 64, stays with that shape up to k = 256; 4096^2 and 6144^2 are 5-12 % faster with
  // 128 x 128 tiles from k = 64 on; 2048^2 and 3072 x 6144 with 128 x 64 ones).  Such a launch of
  // whole tiles takes L + r (F + S k) microseconds, r the tiles on the busiest CU over the
  // workgroups a CU holds, with L, F, S per shape fitted to 13 sizes (2048^2 ... 8192^2, flat
  // and tall ones, 3000^2, 5000^2, 7000^2) x k = 16 ... 160 on MI355X: the shape this picks is
  // within 0.7 % of the fastest on average and 6.7 % at worst, where the smallest shape
  // throughout was 3.6 % and 12.4 % behind.
  if (es == 8 && tri == 0 && nkt >= 2 && nkt <= 10 && tiles64 >= 4 * cus) {
    struct Fit { int id, bm, bn, per_cu; double launch, fixed, per_k; };
    const Fit fits[] = {{RTAT_GEMM_T64x64, 64, 64, 4, 1.6, 4.0, 0.1175},
                        {RTAT_GEMM_T128x64, 128, 64, 2, 3.7, 4.1, 0.108},
                        {RTAT_GEMM_T128x128, 128, 128, 2, 6.1, 9.0, 0.200},
                        {RTAT_GEMM_T256x128, 256, 128, 1, 5.6, 9.3, 0.2185}};
    int pick = RTAT_GEMM_T64x64;
    double least = 0.0;
    for (const Fit& f : fits) {
      const long tiles = (long)((m + f.bm - 1) / f.bm) * ((n + f.bn - 1) / f.bn);
      const double r = (double)((tiles + cus - 1) / cus) / (double)f.per_cu;
      const double us = f.launch + r * (f.fixed + f.per_k * (double)k);
      if (least == 0.0 || us < least) {
        least = us;
        pick = f.id;
      }
    }
    return {pick, false};
  }
  if (nkt <= 8 && tiles64 >= (tri == 0 ? 4 : 8) * cus &&
      (nkt <= 1 || tiles64 <= (tri == 0 ? 48 : 96) * cus))
    return {RTAT_GEMM_T64x64, can_split};
  // Between one 64 x 64 tile for every second CU and one for each, and a k of at most 32 panels:
  // every tile whole.  The model below agrees nearly everywhere in that range, and where it
  // does not - it charges a workgroup alone on its CU more than such a short one costs - the
  // slices it chose lost by a fifth: 512 x 1024 x 256 14.5 us in two slices a tile against 11.3
  // whole, 512 x 1024 x 512 23.0 (128 x 64 tiles in four slices) against 19.3, 640 x 1024 x 512 23.8
  // (three slices) against 19.5.
  if (tri == 0 && tail_mode != RTAT_TAIL_SPLIT && tiles64 * 2 >= cus && tiles64 <= cus && nkt <= 32)
    return {RTAT_GEMM_T64x64, false};
  // More 64 x 64 tiles than CUs but at most one 128 x 64 tile for each, a k of at most 20 panels
  // and an m of whole 128-row tiles: the 128 x 64 shape, every tile whole - half as many
  // workgroups to dispatch for a launch that lasts 12 to 24 us.  3-5 % ahead of the 64 x 64 shape
  // at k = 128 ... 320 over eight shapes (896 x 1536 x 256 19.1 against 19.8 us, 1024 x 2048 x 128 12.6 /
  // 13.2, 640 x 2048 x 256 19.0 / 19.7); from k = 384 on the 64 x 64 shape with its odd tiles cut in
  // two or three is ahead (24.8 against 26.7), and with an m that leaves a partial tile row it is
  // ahead throughout (1100 x 1300 x 128: 14.2 against 15.8), as with half-empty tile columns
  // (32768 x 32 x 256: 22.8 against 24.7).
  {
    const long tiles128x64 = (long)((m + 127) / 128) * ((n + 63) / 64);
    if (tri == 0 && tail_mode != RTAT_TAIL_SPLIT && nkt <= 20 && m % 128 == 0 && n % 64 == 0 &&
        tiles64 > cus && tiles128x64 <= cus)
      return {RTAT_GEMM_T128x64, false};
  }
  // One 128 x 128 tile for (nearly) every CU and a long k: each tile whole, a workgroup alone on
  // its CU.  Half as many waves as the 128 x 64 shape needs to fill the CUs and no trip
  // through scratch: measured 3-7 % ahead of what the model below chooses (8192 x 512 x 8192 926
  // against 976-995 us, 2048 x 2048 x 8192 924 / 956, 1024 x 4096 x 16384 1856 / 1958, 4096 x 1024 x
  // 4096 466 / 480, 2048^3 237 / 244); with a quarter of the CUs empty it loses (3072 x 1024 x 8192
  // 922 against 745 us).
  {
    const long tiles128 = (long)((m + 127) / 128) * ((n + 127) / 128);
    // ... provided the tiles are (nearly) full: 32768 x 64 x 4096 is 256 such tiles as well, each
    // half empty, and took 472 us this way against 282 with 128 x 64 tiles.
    const bool full_tiles = (long)m * n * 10 >= tiles128 * 128 * 128 * 9;
    if (tri == 0 && tail_mode != RTAT_TAIL_SPLIT && tiles128 <= cus && tiles128 * 20 >= cus * 19 &&
        nkt >= 128 && full_tiles)
      return {RTAT_GEMM_T128x128, false};
  }
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
    double second_launch = 0.0;  // of the pieces of a subdivided tail: some 4 us, as for slices
    if (tail > 0) {
      if (full >= 1 && tail_mode != RTAT_TAIL_WHOLE &&
          subdivide_tail(c.bm, c.bn, c.per_cu, tail, cus)) {
        rounds += (double)tail / (double)slots * c.rate / SUB_RATE + 0.03;
        second_launch = 4e-6 * 2.4e9 * (512.0 / es);
      } else {
        const long per_cu_tail = (tail + cus - 1) / cus;  // workgroups a CU holds in the tail
        // Fewer workgroups than a CU can hold share it less efficiently: nothing runs while
        // one sits in its barrier, prologue or epilogue.  For the shapes of 64 x 64 waves that
        // is a cost per tile rather than per k - a lone 128 x 128 workgroup per CU ran
        // 8192 x 512 x 8192 at 74.3 TFLOP/s (925 us whole, 940 us cut in two with the sums
        // added afterwards) - so their surcharge fades with k from 1024 on (12288 x 1000 x 2048
        // 861 -> 705 us, 12288 x 512 x 4096 737 -> 716, 16384 x 768 x 2048 714 -> 697, 6144 x 2048 x
        // 4096 1410 -> 1384; with the 128 x 64 shape included 12288 x 2560 x 3000 and 16384 x 640 x
        // 4096 lost 2 %).
        const double alone =
            (c.bm * c.bn >= 128 * 128 && k > 1024) ? 1.0 + 0.15 * 1024.0 / (double)k : 1.15;
        rounds += (double)per_cu_tail / (double)c.per_cu * (per_cu_tail < c.per_cu ? alone : 1.0);
        lone = full == 0 && per_cu_tail < 2 && c.per_cu > 1;
      }
    }
    double cost =
        rounds * area * ((double)k / (c.rate * (lone ? 0.975 : 1.0)) + (lone ? 400.0 : 230.0)) +
        second_launch;
    bool split = false;
    // ... or cut along K, where the rule allows it: a fraction of a round, plus the slices'
    // trip through scratch (written and read back once at about 4 TB/s) and a second launch
    // of some 4 us; a CU retires 512 / es products per cycle at 2.4 GHz.
    if (tail > 0 && can_split) {
      const SplitPlan plan = split_plan(tiles, cus, c.per_cu, nkt,
                                        tail_mode == RTAT_TAIL_SPLIT ? SPLIT_FORCED : SPLIT_PRICED, es);
      long slices = plan.slices, more = plan.more;
      clamp_to_room(plan.tiles, slices, more, split_room(c.bm, c.bn, es));
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
        // When every tile is sliced, the slices are short and a CU holds a single one of
        // them, the smallest shape - two workgroups of half the size on that CU, which hide
        // each other's prologues and epilogues - is ahead of what its rate says.  Over 117
        // problems of 18 to 72 tiles of 128 x 64 and k = 768 ... 8192 the 64 x 64 shape with the
        // same slice count ran 5 % faster at 300 k a slice, 3.5 % at 600, 1 % at 1000 and level
        // or behind from 1200 on; where the slices fill the slots of either shape (768 x 768 x
        // 3072 ... 8192) the two are level at every k.
        double short_slices = 1.0;
        if (whole == 0 && on_cu == 1 && c.per_cu == 2) {
          const double ks = (double)k / (double)slices;
          if (ks < 1200.0) short_slices += 0.08 * (1.0 - ks / 1200.0);
        }
        const double cut =
            (whole_rounds + sliced * short_slices) * area * ((double)k / c.rate + 230.0) + trip;
        if (cut < cost || tail_mode == RTAT_TAIL_SPLIT) {
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


}  // namespace rtat_native
