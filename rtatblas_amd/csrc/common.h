// Internal declarations shared by the kernel translation units of librtat_native.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <vector>
#include "rtat_measure.h"
#include "rtat_native.h"
#include "trsm_plan.h"

struct rtat_native_handle {
  hipStream_t stream = nullptr;
  int device = 0;
  int compute_units = 0;
  double clock_hz = 0.0;
  double mem_bytes_per_s = 0.0;
  size_t max_dyn_lds = 0;
  // TRSM scratch: either lent by the caller or owned (grown on demand).
  void* user_ws = nullptr;
  size_t user_ws_bytes = 0;
  void* own_ws = nullptr;
  size_t own_ws_bytes = 0;
  // Owned blocks that a larger one has replaced.  Work already enqueued, or a graph captured
  // earlier, may still name them, so they live until the handle is destroyed.
  std::vector<void*> retired_ws;
  // GEMM tail-splitting scratch (slices of the last tiles), owned, allocated with the handle.
  void* split_ws = nullptr;
  bool split_ws_failed = false;
  // Device address of the library's static scratch array on this handle's device
  // (rtat_dtrsm_static), nullptr if it could not be looked up.
  void* static_ws = nullptr;
  // What the last GEMM-core launch on this handle did (rtat_last_launch).
  rtat_launch_info_t last = {};
  int last_bm = 0, last_bn = 0;  // its tile shape; spelled into last.tile when asked for
};

namespace rtat_native {

constexpr int MAX_DEVICES = 64;  // per-device bookkeeping of kernel attributes

inline bool valid_op(int op) { return op == RTAT_OP_N || op == RTAT_OP_T; }
inline bool valid_fill(int f) { return f == RTAT_FILL_UPPER || f == RTAT_FILL_LOWER; }
inline bool valid_diag(int d) { return d == RTAT_DIAG_NON_UNIT || d == RTAT_DIAG_UNIT; }
inline bool valid_side(int s) { return s == RTAT_SIDE_LEFT || s == RTAT_SIDE_RIGHT; }

// The kernel-options word of the *_ex entry points, taken apart.  False when a field is out
// of range or a bit outside the three fields is set.
struct KernelOptions {
  int tile, tail, panel;
};
inline bool decode_options(int word, KernelOptions& o) {
  if (word < 0 || (word >> 16) != 0) return false;
  o.tile = RTAT_KERNEL_OPTIONS_TILE(word);
  o.tail = RTAT_KERNEL_OPTIONS_TAIL(word);
  o.panel = RTAT_KERNEL_OPTIONS_PANEL(word);
  return o.tile < RTAT_GEMM_VARIANT_COUNT && o.tail < RTAT_TAIL_MODE_COUNT &&
         o.panel < RTAT_PANEL_COUNT;
}

inline rtat_status_t launch_status() {
  return hipGetLastError() == hipSuccess ? RTAT_STATUS_SUCCESS : RTAT_STATUS_EXECUTION_FAILED;
}

// Allocation on the handle's device whatever device is current on the calling thread.
inline hipError_t malloc_on_device(int device, void** p, size_t bytes) {
  int cur = -1;
  if (hipGetDevice(&cur) != hipSuccess) cur = -1;
  if (cur != device && hipSetDevice(device) != hipSuccess) return hipErrorInvalidDevice;
  const hipError_t e = hipMalloc(p, bytes);
  if (cur != device && cur >= 0) (void)hipSetDevice(cur);
  return e;
}

// True while `s` records into a graph.  Device memory cannot be allocated or freed then (the
// runtime would refuse and invalidate the capture), so the library's lazy allocations are
// skipped: a call that needs scratch it does not have yet reports RTAT_STATUS_ALLOC_FAILED,
// and GEMM tails are not split.  A query that fails counts as capturing.
inline bool stream_capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return true;
  }
  return st != hipStreamCaptureStatusNone;
}

// Scratch of at least `bytes` for the current call, or nullptr when it cannot be had.
void* acquire_workspace(rtat_native_handle* h, size_t bytes);

// Allocate the handle's scratch for GEMM tail slices if it has none yet (gemm.hip).
void prepare_split_workspace(rtat_native_handle* h);

// Once-per-device set-up of a kernel (its dynamic LDS limit): true when `setup` has succeeded
// on this device before or succeeds now.  Safe to call from several host threads; a second
// thread may repeat a set-up that is in flight, which is harmless.
struct PerDeviceOnce {
  std::atomic<bool> done[MAX_DEVICES] = {};
  template <class F>
  bool operator()(int device, F setup) {
    const int d = (device >= 0 && device < MAX_DEVICES) ? device : 0;
    if (done[d].load(std::memory_order_acquire)) return true;
    if (!setup()) return false;
    done[d].store(true, std::memory_order_release);
    return true;
  }
};

// ---- kernel launchers (one per translation unit) -------------------------------------

// C = alpha*op(A)*op(B) + beta*C on the MFMA core (T = double or float).  tri: 0 full,
// 1 lower, 2 upper (only that triangle of a square C is computed and written).
template <typename T>
rtat_status_t launch_gemm(rtat_native_handle* h, bool ta, bool tb, int m, int n, int k, T alpha,
                          const T* A, int lda, const T* B, int ldb, T beta, T* C, int ldc,
                          int tri, int variant);

inline rtat_status_t launch_dgemm(rtat_native_handle* h, bool ta, bool tb, int m, int n, int k,
                                  double alpha, const double* A, int lda, const double* B,
                                  int ldb, double beta, double* C, int ldc, int tri,
                                  int variant) {
  return launch_gemm<double>(h, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, tri,
                             variant);
}

template <typename T>
rtat_status_t launch_geam(rtat_native_handle* h, bool ta, bool tb, int m, int n, T alpha,
                          const T* A, int lda, T beta, const T* B, int ldb, T* C, int ldc);

template <typename T>
rtat_status_t launch_fill(rtat_native_handle* h, T* A, int m, int n, int ld, uint64_t seed,
                          int kind);

// Two copies / transposes in one launch (rtat_dmove_pair / rtat_smove_pair).
template <typename T>
rtat_status_t launch_move_pair(rtat_native_handle* h, const rtat_move_t* first,
                               const rtat_move_t* second);

// Plain streaming kernel over the caller's buffers (rtat_hbm_probe).
rtat_status_t launch_probe(rtat_native_handle* h, int kind, const void* src, void* dst,
                           size_t bytes);

// In-place triangular solve (T = double or float); takes trsm_workspace_bytes(na) of
// scratch from acquire_workspace.
template <typename T>
rtat_status_t launch_trsm(rtat_native_handle* h, bool left, bool lower, bool trans, bool unit,
                          int m, int n, T alpha, const T* A, int lda, T* B, int ldb,
                          int variant);

// ---- counter-based generator (identical on host and device) --------------------------

__host__ __device__ inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// u in [0,1) with 53 random bits, a function of (seed, i, j) only.
__host__ __device__ inline double unit_uniform(uint64_t seed, uint32_t i, uint32_t j) {
  uint64_t z = mix64(seed * 0x9E3779B97F4A7C15ull + (((uint64_t)j << 32) | (uint64_t)i));
  return (double)(z >> 11) * (1.0 / 9007199254740992.0);
}

}  // namespace rtat_native
