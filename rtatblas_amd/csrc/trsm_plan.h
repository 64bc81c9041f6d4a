// Blocking of the triangular solve (trsm.hip): block order, panel heights, scratch size, and
// the order in which a block of the system matrix is laid out for the panel kernel.  Plain
// integer arithmetic that also compiles for the host alone: the static scratch of
// rtat_dtrsm_static is sized from it (api.hip) and a CPU test checks the layout map
// (tests/cpp).
#pragma once
#include <stddef.h>

#ifndef RTAT_HD
#if defined(__HIPCC__)
#define RTAT_HD __host__ __device__
#else
#define RTAT_HD
#endif
#endif

namespace rtat_native {

constexpr int NB = 128;  // order of the diagonal blocks that are inverted
// Rows of the triangular dimension solved per launch of the panel kernel: 512, or 1024, which
// saves a level of GEMM updates and is taken as soon as the panel kernel has workgroups for
// more than half the CUs.
constexpr int PANEL_SHORT = 4 * NB;
constexpr int PANEL_TALL = 8 * NB;
// Off-diagonal blocks of a panel of `blocks` diagonal blocks.
RTAT_HD constexpr int panel_pairs(int blocks) { return blocks * (blocks - 1) / 2; }
// Scratch elements of a solve with a triangular matrix of order na and the given panel
// height: one NB x NB inverse per diagonal block, then the off-diagonal blocks of every panel.
constexpr size_t trsm_scratch_elems(int na, int panel, size_t* packed_offset) {
  const size_t nblk = (size_t)(na + NB - 1) / NB, npanel = (size_t)(na + panel - 1) / panel;
  if (packed_offset != nullptr) *packed_offset = nblk * NB * NB;
  return (nblk + npanel * (size_t)panel_pairs(panel / NB)) * NB * NB;
}

// Fragment order of a 128 x 128 block of M for the 16x16x4 MFMAs of trsm_panel_kernel: wave
// v = row / 16 of a workgroup takes MFMA step group g = k / 4E (E = elements per 16 bytes) with
// one 16-byte load per lane, lane = 16 kq + row % 16 holding k = 4E g + E kq + e, e = 0 .. E-1;
// the 64 lanes' loads of one group are 1 KiB in a row.
template <class T>
RTAT_HD inline int frag_offset(int row, int k) {
  constexpr int E = 16 / (int)sizeof(T), NGRP = NB / (4 * E);
  const int v = row >> 4, r16 = row & 15, g = k / (4 * E), kq = (k % (4 * E)) / E, e = k % E;
  return ((v * NGRP + g) * 64 + 16 * kq + r16) * E + e;
}

}  // namespace rtat_native
