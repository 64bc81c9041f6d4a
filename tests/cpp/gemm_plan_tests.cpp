// CPU sweep of the GEMM / SYRK launch planning (rtatblas_amd/csrc/gemm_plan.h): the kernel
// indexes its split scratch, its K slices and its tiles by what these functions return, so a
// rule that breaks an invariant would be an out-of-bounds access on the device.  Every
// combination of tile shape, element size, CU count, triangle mode and split mode is swept
// over a grid of problem shapes; no device is touched.
#include <gemm_plan.h>
#include <trsm_plan.h>

#include <set>
#include <utility>
#include <vector>

#include "mini_test.h"

using namespace rtat_native;

namespace {

struct Shape {
  int id, bm, bn, per_cu;
};
const Shape SHAPES[] = {{RTAT_GEMM_T256x128, 256, 128, 1}, {RTAT_GEMM_T128x128, 128, 128, 2},
                        {RTAT_GEMM_T128x64, 128, 64, 2}, {RTAT_GEMM_T64x64, 64, 64, 4},
                        {GEMM_SHAPE_T32x32, 32, 32, 4}};
const long CU_COUNTS[] = {8, 64, 104, 228, 256, 304, 320};
const int SIZES[] = {1, 63, 64, 65, 200, 512, 1000, 1152, 1600, 2560, 3072, 3584, 4099, 6151,
                     8192, 10007};
const int DEPTHS[] = {1, 15, 16, 100, 128, 700, 2048, 8192, 65536};

// The tiles the kernel must compute: all of them, or those touching the wanted triangle.
bool tile_wanted(int tri, int i, int j, int bm, int bn) {
  const long m0 = (long)i * bm, n0 = (long)j * bn;
  if (tri == 1) return n0 <= m0 + bm - 1;      // some element with row >= col
  if (tri == 2) return n0 + bn - 1 >= m0;      // some element with row <= col
  return true;
}

long count_wanted(int tri, int tiles_m, int tiles_n, int bm, int bn) {
  long c = 0;
  for (int i = 0; i < tiles_m; ++i)
    for (int j = 0; j < tiles_n; ++j) c += tile_wanted(tri, i, j, bm, bn);
  return c;
}

}  // namespace

TEST(GemmPlan, Invariants_Over_A_Sweep_Of_Shapes, false) {
  long points = 0, split_points = 0, sub_points = 0;
  for (const Shape& sh : SHAPES)
    for (int es : {8, 4})
      for (long cus : CU_COUNTS)
        for (int tri : {0, 1, 2})
          for (int mode : {SPLIT_NEVER, SPLIT_STATIC, SPLIT_PRICED, SPLIT_FORCED, SPLIT_WHOLE})
            for (int m : SIZES)
              for (int n : SIZES) {
                if (tri != 0 && m != n) continue;
                for (int k : DEPTHS) {
                  const int bk = 128 / es;
                  const LaunchPlan p = plan_launch(m, n, k, tri, sh.bm, sh.bn, bk, sh.per_cu, es,
                                                   cus, mode, true, true);
                  ++points;
                  const long nkt = (k + bk - 1) / bk;
                  CHECK_EQ(p.tiles_m, (m + sh.bm - 1) / sh.bm);
                  CHECK_EQ(p.tiles_n, (n + sh.bn - 1) / sh.bn);
                  if (p.tiles_m <= 64 && p.tiles_n <= 64)
                    CHECK_EQ(p.tiles, count_wanted(tri, p.tiles_m, p.tiles_n, sh.bm, sh.bn));
                  CHECK(p.tiles >= 1);
                  if (mode == SPLIT_NEVER || mode == SPLIT_WHOLE) CHECK_EQ(p.split_tiles, 0);
                  if (mode == SPLIT_WHOLE) {  // one launch, every tile whole
                    CHECK_EQ(p.sub_count, 0L);
                    CHECK_EQ(p.grid, p.tiles);
                  }
                  if (mode == SPLIT_FORCED) {  // a superset of what the fixed rule cuts
                    const LaunchPlan q = plan_launch(m, n, k, tri, sh.bm, sh.bn, bk, sh.per_cu,
                                                     es, cus, SPLIT_STATIC, true, true);
                    if (q.split_tiles > 0) CHECK(p.split_tiles > 0);
                  }
                  if (p.sub_count > 0) {
                    ++sub_points;
                    CHECK_EQ(p.split_tiles, 0);
                    CHECK_EQ(p.lead + p.sub_count, p.tiles);
                    CHECK_EQ(p.grid, p.lead);
                    CHECK(p.lead >= 1);
                    const long pieces = (long)(sh.bm / 64) * (sh.bn / 64);
                    CHECK_EQ(p.sub_grid % (XCDS * pieces), 0L);
                    CHECK(p.sub_grid / pieces >= p.sub_count);          // every big tile has its group
                    CHECK(p.sub_grid / pieces < p.sub_count + XCDS);    // and at most 7 empty ones
                    continue;
                  }
                  CHECK_EQ(p.whole + p.split_tiles, p.tiles);
                  CHECK_EQ(p.grid, p.whole + (long)p.split_tiles * p.split_s + p.split_more);
                  if (p.split_tiles == 0) {
                    CHECK_EQ(p.split_s, 1);
                    CHECK_EQ(p.split_more, 0);
                    CHECK_EQ(p.reduce_grid, 0L);
                    continue;
                  }
                  ++split_points;
                  const long slots_used = (long)p.split_tiles * p.split_s + p.split_more;
                  CHECK(p.split_s >= 2);
                  CHECK(p.split_more >= 0 && p.split_more <= p.split_tiles);
                  CHECK(slots_used <= split_room(sh.bm, sh.bn, es));    // scratch is not overrun
                  CHECK(p.split_s + (p.split_more > 0 ? 1 : 0) <= nkt);  // no slice without a panel
                  CHECK(p.split_tiles <= p.tiles);
                  CHECK_EQ(p.reduce_grid, (long)p.split_tiles * (sh.bn / 8));
                  // slot numbering: consecutive, in tile order, the longer-sliced tiles last
                  long next = 0;
                  for (int t = 0; t < p.split_tiles; ++t) {
                    int count;
                    long first;
                    slices_of_tile(t, p.split_tiles, p.split_s, p.split_more, count, first);
                    CHECK_EQ(first, next);
                    CHECK_EQ(count, p.split_s + (t >= p.split_tiles - p.split_more ? 1 : 0));
                    next += count;
                  }
                  CHECK_EQ(next, slots_used);
                  // K slices: a partition of the panels, none empty
                  for (int slices : {p.split_s, p.split_s + 1}) {
                    long at = 0;
                    for (int sl = 0; sl < slices && slices <= nkt; ++sl) {
                      long first, count;
                      slice_panels(nkt, slices, sl, first, count);
                      CHECK_EQ(first, at);
                      CHECK(count >= 1);
                      at += count;
                    }
                    if (slices <= nkt) CHECK_EQ(at, nkt);
                  }
                }
              }
  std::cout << "    " << points << " plans, " << split_points << " with K slices, " << sub_points
            << " subdivided" << std::endl;
  CHECK(points > 300000);
  CHECK(split_points > 10000);
  CHECK(sub_points > 100);
}

TEST(GemmPlan, Scratch_Room_Is_Respected_When_It_Is_Tight, false) {
  // Problems of few huge-K tiles on many CUs want more slices than a small room holds: the
  // clamp has to bring them down, for the launcher and for the heuristic alike.
  for (long room : {1L, 2L, 3L, 7L, 64L, 511L}) {
    for (long tiles : {1L, 2L, 3L, 5L, 100L}) {
      for (long want : {2L, 3L, 64L, 512L}) {
        long s = want, more = tiles / 2;
        clamp_to_room(tiles, s, more, room);
        CHECK(tiles * s + more <= room || s < 2 || (s == want && more == tiles / 2));
        if (tiles * want + tiles / 2 > room) {
          CHECK_EQ(more, 0L);
          CHECK(tiles * s <= room || s == 0);
        }
      }
    }
  }
}

TEST(GemmPlan, Workgroup_Ids_Cover_Every_Tile_Once, false) {
  // logical_of_workgroup is a permutation of [0, whole); tile_of_logical maps [0, tiles)
  // one-to-one onto the wanted tiles, for full and triangular C and every tile shape.
  for (int whole : {1, 2, 7, 8, 9, 63, 64, 65, 511, 1000, 4097}) {
    std::vector<char> seen(whole, 0);
    for (int wg = 0; wg < whole; ++wg) {
      const int l = logical_of_workgroup(wg, whole);
      CHECK(l >= 0 && l < whole);
      if (l >= 0 && l < whole) {
        CHECK(!seen[l]);
        seen[l] = 1;
      }
    }
  }
  for (const Shape& sh : SHAPES)
    for (int tri : {0, 1, 2})
      for (int m : {1, 64, 65, 200, 1000, 1152, 3000, 4099, 8192, 12288})
        for (int n : {1, 100, 129, 1000, 4099, 8192}) {
          if (tri != 0 && m != n) continue;
          const int tm = (m + sh.bm - 1) / sh.bm, tn = (n + sh.bn - 1) / sh.bn;
          const long tiles = count_wanted(tri, tm, tn, sh.bm, sh.bn);
          std::set<std::pair<int, int>> hit;
          for (long l = 0; l < tiles; ++l) {
            int i, j;
            tile_of_logical((int)l, tm, tn, tri, sh.bm, sh.bn, i, j);
            CHECK(i >= 0 && i < tm && j >= 0 && j < tn);
            CHECK(tile_wanted(tri, i, j, sh.bm, sh.bn));
            hit.insert({i, j});
          }
          CHECK_EQ((long)hit.size(), tiles);
        }
}

TEST(GemmPlan, Subdivision_Ids_Cover_Every_Piece_Once, false) {
  // The second launch of a subdivided tail: workgroup id -> (big tile, piece) as the kernel
  // decodes it; every piece of every leftover tile exactly once, ids past the count idle.
  for (const Shape& sh : SHAPES) {
    const long pieces = (long)(sh.bm / 64) * (sh.bn / 64);
    for (long count : {1L, 7L, 8L, 9L, 100L, 257L}) {
      const long grid = (count + XCDS - 1) / XCDS * pieces * XCDS;
      std::set<std::pair<long, long>> hit;
      for (long wg = 0; wg < grid; ++wg) {
        const long x = wg % XCDS, j = wg / XCDS;
        const long big = (j / pieces) * XCDS + x, piece = j % pieces;
        if (big >= count) continue;
        CHECK(hit.insert({big, piece}).second);
      }
      CHECK_EQ((long)hit.size(), count * pieces);
    }
  }
}

TEST(GemmPlan, Shape_Heuristic_Returns_A_Shape_For_Every_Problem, false) {
  long calls = 0;
  for (long cus : CU_COUNTS)
    for (int es : {8, 4})
      for (int tri : {0, 1, 2})
        for (int m : SIZES)
          for (int n : SIZES) {
            if (tri != 0 && m != n) continue;
            for (int k : DEPTHS)
              for (bool can_split : {false, true})
                for (int tail : {RTAT_TAIL_AUTO, RTAT_TAIL_WHOLE, RTAT_TAIL_SPLIT}) {
                  const Pick pk = pick_variant(cus, m, n, k, 128 / es, es, tri, can_split, tail);
                  ++calls;
                  CHECK(pk.variant >= RTAT_GEMM_T256x128 && pk.variant <= GEMM_SHAPE_T32x32);
                  // the 32 x 32 shape is never asked to cut its tiles
                  CHECK(pk.variant != GEMM_SHAPE_T32x32 || !pk.split);
                  if (tail == RTAT_TAIL_WHOLE || !can_split) CHECK(!pk.split);
                }
          }
  CHECK(calls > 50000);
}

TEST(GemmPlan, Measured_Choices_Of_The_Shape_Heuristic, false) {
  // The choices the rules in front of the cost model were measured for, on 256 CUs in double
  // precision: a regression here means a rule no longer reaches the shapes it was written for.
  auto pick = [](int m, int n, int k, int es = 8) {
    return pick_variant(256, m, n, k, 128 / es, es, 0, true, RTAT_TAIL_AUTO);
  };
  // between one 64 x 64 tile for every second CU and one for each, k <= 32 panels: whole tiles
  for (int k : {256, 384, 512})
    for (auto mn : {std::pair<int, int>(512, 1024), {256, 2048}, {640, 1024}, {768, 1024}}) {
      const Pick p = pick(mn.first, mn.second, k);
      CHECK_EQ(p.variant, (int)RTAT_GEMM_T64x64);
      CHECK(!p.split);
    }
  // more of those tiles than CUs, at most one 128 x 64 tile per CU, short k, whole tile rows
  for (auto mn : {std::pair<int, int>(896, 1536), {1024, 1280}, {640, 2048}, {1024, 2048}}) {
    const Pick p = pick(mn.first, mn.second, 256);
    CHECK_EQ(p.variant, (int)RTAT_GEMM_T128x64);
    CHECK(!p.split);
  }
  CHECK_EQ(pick(1100, 1300, 256).variant, (int)RTAT_GEMM_T64x64);   // a partial tile row
  CHECK(pick(896, 1536, 384).variant != (int)RTAT_GEMM_T128x64 || pick(896, 1536, 384).split);
  // small k on a large C: by the fitted launch time of whole tiles
  CHECK_EQ(pick(3072, 3072, 128).variant, (int)RTAT_GEMM_T64x64);
  CHECK_EQ(pick(6144, 6144, 128).variant, (int)RTAT_GEMM_T128x128);
  CHECK_EQ(pick(4096, 6144, 128).variant, (int)RTAT_GEMM_T128x128);
  CHECK_EQ(pick(3072, 6144, 96).variant, (int)RTAT_GEMM_T128x64);
  CHECK_EQ(pick(3000, 3000, 64).variant, (int)RTAT_GEMM_T64x64);
  CHECK_EQ(pick(8192, 8192, 128).variant, (int)RTAT_GEMM_T128x128);
  CHECK_EQ(pick(4096, 4096, 16).variant, (int)RTAT_GEMM_T64x64);    // a single panel
  CHECK_EQ(pick(4096, 4096, 128, 4).variant, (int)RTAT_GEMM_T64x64);  // single precision: the old rule
  // slices: three a tile for the 64 x 64 shape at 40 ... 64 panels when they fill 3/4 of the CUs
  const SplitPlan three = split_plan(144, 256, 4, 48, SPLIT_PRICED, 8);
  CHECK_EQ(three.tiles, 144L);
  CHECK_EQ(three.slices, 3L);
  CHECK(split_plan(144, 256, 4, 32, SPLIT_PRICED, 8).slices != 3);
  CHECK(split_plan(144, 256, 4, 96, SPLIT_PRICED, 8).slices != 3);
  CHECK_EQ(split_plan(144, 256, 4, 48, SPLIT_PRICED, 4).slices, 3L);
  CHECK(split_plan(144, 256, 4, 64, SPLIT_PRICED, 4).slices != 3);
  CHECK(split_plan(196, 256, 4, 48, SPLIT_PRICED, 8).slices != 2);   // two a tile never by this rule
  // the odd tiles beyond one per CU are not cut below 20 panels
  CHECK_EQ(split_plan(336, 256, 4, 16, SPLIT_STATIC, 8).tiles, 0L);
  const SplitPlan odd = split_plan(336, 256, 4, 24, SPLIT_STATIC, 8);
  CHECK_EQ(odd.tiles, 80L);
  CHECK(odd.slices >= 2);
  // 768^3: the 64 x 64 shape in three slices a tile
  const Pick cube = pick(768, 768, 768);
  CHECK_EQ(cube.variant, (int)RTAT_GEMM_T64x64);
  CHECK(cube.split);
  // one 128 x 128 tile per CU and a long k: that shape whole - unless the tiles are half empty
  CHECK_EQ(pick(8192, 512, 8192).variant, (int)RTAT_GEMM_T128x128);
  CHECK(!pick(8192, 512, 8192).split);
  CHECK(pick(32768, 64, 4096).variant != (int)RTAT_GEMM_T128x128);
  CHECK(pick(64, 32768, 4096).variant != (int)RTAT_GEMM_T128x128);
  // every tile sliced, short slices, one 128 x 64 slice per CU: the 64 x 64 shape
  CHECK_EQ(pick(384, 768, 2048).variant, (int)RTAT_GEMM_T64x64);
  CHECK_EQ(pick(512, 640, 1536).variant, (int)RTAT_GEMM_T64x64);
}

template <class T>
static void check_fragment_order() {
  // frag_offset is one-to-one from the 128 x 128 elements of a block onto its 16384 slots, and
  // the slot the panel kernel's lane l of wave v reads as element e of step group g holds row
  // 16 v + l % 16 at k = 4E g + E (l / 16) + e.
  constexpr int E = 16 / (int)sizeof(T), NGRP = NB / (4 * E);
  std::vector<char> seen(NB * NB, 0);
  for (int row = 0; row < NB; ++row)
    for (int k = 0; k < NB; ++k) {
      const int o = frag_offset<T>(row, k);
      CHECK(o >= 0 && o < NB * NB);
      if (o >= 0 && o < NB * NB) {
        CHECK(!seen[o]);
        seen[o] = 1;
      }
    }
  for (int v = 0; v < NB / 16; ++v)
    for (int g = 0; g < NGRP; ++g)
      for (int l = 0; l < 64; ++l)
        for (int e = 0; e < E; ++e)
          CHECK_EQ(frag_offset<T>(16 * v + l % 16, 4 * E * g + E * (l / 16) + e),
                   ((v * NGRP + g) * 64 + l) * E + e);
}

TEST(TrsmPlan, Fragment_Order_Is_The_Panel_Kernels_Read_Order, false) {
  check_fragment_order<double>();
  check_fragment_order<float>();
}

TEST(TrsmPlan, Scratch_Holds_The_Inverses_And_The_Blocks_Of_Every_Panel, false) {
  // by hand: order 4096 with 1024-row panels = 32 inverses + 4 x 28 blocks; the short layout of
  // the same order 32 + 8 x 6; a ragged order rounds both counts up
  size_t off = 0;
  CHECK_EQ(trsm_scratch_elems(4096, PANEL_TALL, &off), (size_t)(32 + 4 * 28) * NB * NB);
  CHECK_EQ(off, (size_t)32 * NB * NB);
  CHECK_EQ(trsm_scratch_elems(4096, PANEL_SHORT, nullptr), (size_t)(32 + 8 * 6) * NB * NB);
  CHECK_EQ(trsm_scratch_elems(1025, PANEL_TALL, nullptr), (size_t)(9 + 2 * 28) * NB * NB);
  CHECK_EQ(trsm_scratch_elems(1, PANEL_SHORT, nullptr), (size_t)(1 + 6) * NB * NB);
}
