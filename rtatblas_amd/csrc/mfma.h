// Element-type traits of the 16x16x4 MFMA kernels (double and float) and the vector types
// they move data with.
#pragma once
#include <hip/hip_runtime.h>

namespace rtat_native {

typedef double d2_t __attribute__((ext_vector_type(2)));
typedef double d4_t __attribute__((ext_vector_type(4)));
typedef float f2_t __attribute__((ext_vector_type(2)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef unsigned u2_t __attribute__((ext_vector_type(2)));
typedef unsigned u4_t __attribute__((ext_vector_type(4)));

// Per element type: E = elements per 16-byte vector, the 16x16x4 MFMA and the place of its
// result: accumulator register r of lane l holds D[acc_row(r, l)][l % 16].
template <class T> struct Elem;
template <> struct Elem<double> {
  static constexpr int E = 2;
  typedef d4_t acc_t;
  __device__ static inline acc_t mfma(double a, double b, acc_t c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  __device__ static inline int acc_row(int r, int lane) { return 4 * r + (lane >> 4); }
};
template <> struct Elem<float> {
  static constexpr int E = 4;
  typedef f4_t acc_t;
  __device__ static inline acc_t mfma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  __device__ static inline int acc_row(int r, int lane) { return 4 * (lane >> 4) + r; }
};

// N elements of T as one naturally aligned vector (N * sizeof(T) = 8 or 16 bytes, or N = 1).
template <class T, int N> struct VecOf { typedef T type __attribute__((ext_vector_type(N))); };
template <class T> struct VecOf<T, 1> { typedef T type; };

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

}  // namespace rtat_native
