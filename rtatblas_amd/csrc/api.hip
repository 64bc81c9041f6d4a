// extern "C" entry points of librtat_native (declared in include/rtat_native.h): argument
// checking, host-pointer scalars read by value, dispatch to the kernel launchers.
#include <new>
#include "common.h"

#include <stdio.h>

#include <mutex>

using namespace rtat_native;

// Scratch of rtat_dtrsm_static: one array per GPU, part of the library's device image, held
// until the process ends.  Sized for a triangular matrix of order RTAT_DTRSM_STATIC_MAX_ORDER
// in either panel layout.  Host code never passes this name anywhere: it stands for the
// array only inside device code; the device address comes from hipGetSymbolAddress, once per
// device, in static_scratch_of below.
constexpr size_t scratch_bytes_for(int order) {
  const size_t tall = rtat_native::trsm_scratch_elems(order, rtat_native::PANEL_TALL, nullptr);
  const size_t low = rtat_native::trsm_scratch_elems(order, rtat_native::PANEL_SHORT, nullptr);
  return (tall > low ? tall : low) * sizeof(double) + 256;
}
constexpr size_t STATIC_SCRATCH_BYTES = scratch_bytes_for(RTAT_DTRSM_STATIC_MAX_ORDER);
static_assert(STATIC_SCRATCH_BYTES <= ((size_t)32 << 20), "the static scratch is meant to stay modest");
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace rtat_native {

size_t trsm_workspace_bytes(int na);

// Device address of this device's copy of `scratch`, looked up the first time a handle is
// created on the device (with that device current) and remembered.  nullptr if the lookup
// failed.
static void* static_scratch_of(int device) {
  static std::mutex guard;
  static void* address[MAX_DEVICES] = {};
  static bool asked[MAX_DEVICES] = {};
  if (device < 0 || device >= MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(guard);
  if (!asked[device]) {
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess || cur != device) {
      (void)hipGetLastError();
      return nullptr;  // only rtat_create asks first, and it asks for the current device
    }
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      ptr = nullptr;
    }
    address[device] = ptr;
    asked[device] = true;
  }
  return address[device];
}

// Handle-owned scratch grows by allocating a new block (at least twice the old size, so the
// retired blocks of a handle never add up to more than its current one).  The old block is
// not freed here: kernels already enqueued, on this stream or on one the handle served
// before, and graphs captured earlier may still name it.  It is parked on the handle and
// freed by rtat_destroy.  Nothing synchronises.
void* acquire_workspace(rtat_native_handle* h, size_t bytes) {
  if (bytes == 0) return h->user_ws ? h->user_ws : h->own_ws;
  if (h->user_ws != nullptr) return h->user_ws_bytes >= bytes ? h->user_ws : nullptr;
  if (h->own_ws_bytes < bytes) {
    if (stream_capturing(h->stream)) return nullptr;
    size_t want = 2 * h->own_ws_bytes;
    if (want < bytes) want = bytes;
    void* p = nullptr;
    if (malloc_on_device(h->device, &p, want) != hipSuccess) {
      (void)hipGetLastError();
      want = bytes;
      if (malloc_on_device(h->device, &p, want) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
      }
    }
    if (h->own_ws != nullptr) {
      try {
        h->retired_ws.push_back(h->own_ws);
      } catch (...) {  // no room to remember the old block: keep using it
        (void)hipFree(p);
        return nullptr;
      }
    }
    h->own_ws = p;
    h->own_ws_bytes = want;
  }
  return h->own_ws;
}

}  // namespace rtat_native

#define RTAT_CHECK_HANDLE(h) \
  if ((h) == nullptr) return RTAT_STATUS_HANDLE_IS_NULLPTR

extern "C" {

rtat_status_t rtat_create(rtat_handle_t* handle) {
  if (handle == nullptr) return RTAT_STATUS_INVALID_VALUE;
  *handle = nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return RTAT_STATUS_NOT_INITIALIZED;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    (void)hipGetLastError();
    return RTAT_STATUS_NOT_INITIALIZED;
  }
  rtat_native_handle* h = new (std::nothrow) rtat_native_handle();
  if (h == nullptr) return RTAT_STATUS_ALLOC_FAILED;
  h->device = dev;
  h->compute_units = prop.multiProcessorCount;
  h->clock_hz = (double)prop.clockRate * 1e3;
  h->mem_bytes_per_s = 2.0 * (double)prop.memoryClockRate * 1e3 * (double)prop.memoryBusWidth / 8.0;
  h->max_dyn_lds = prop.sharedMemPerBlock;
  // The scratch for GEMM / SYRK tail slices comes with the handle, so that no compute call
  // ever allocates it inside a caller's event pair.  Without it tails are computed unsplit.
  prepare_split_workspace(h);
  h->static_ws = static_scratch_of(dev);
  *handle = h;
  return RTAT_STATUS_SUCCESS;
}

rtat_status_t rtat_destroy(rtat_handle_t h) {
  RTAT_CHECK_HANDLE(h);
  if (h->own_ws != nullptr || h->split_ws != nullptr || !h->retired_ws.empty()) {
    // Freeing device memory while a stream records into a graph would invalidate the capture:
    // refuse, and leave the handle as it is.
    if (stream_capturing(h->stream)) return RTAT_STATUS_NOT_SUPPORTED;
    // Work still in flight on any stream of the handle's device may name the blocks: let that
    // device drain first, whichever device is current on this thread.
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess) cur = -1;
    if (cur != h->device) (void)hipSetDevice(h->device);
    (void)hipDeviceSynchronize();
    if (h->own_ws != nullptr) (void)hipFree(h->own_ws);
    for (void* p : h->retired_ws) (void)hipFree(p);
    if (h->split_ws != nullptr) (void)hipFree(h->split_ws);
    if (cur != h->device && cur >= 0) (void)hipSetDevice(cur);
    (void)hipGetLastError();
  }
  delete h;
  return RTAT_STATUS_SUCCESS;
}

rtat_status_t rtat_set_stream(rtat_handle_t h, rtat_stream_t stream) {
  RTAT_CHECK_HANDLE(h);
  h->stream = static_cast<hipStream_t>(stream);
  return RTAT_STATUS_SUCCESS;
}

rtat_status_t rtat_get_stream(rtat_handle_t h, rtat_stream_t* stream) {
  RTAT_CHECK_HANDLE(h);
  if (stream == nullptr) return RTAT_STATUS_INVALID_VALUE;
  *stream = static_cast<rtat_stream_t>(h->stream);
  return RTAT_STATUS_SUCCESS;
}

rtat_status_t rtat_set_workspace(rtat_handle_t h, void* device_ptr, size_t bytes) {
  RTAT_CHECK_HANDLE(h);
  if ((device_ptr == nullptr) != (bytes == 0)) return RTAT_STATUS_INVALID_VALUE;
  h->user_ws = device_ptr;
  h->user_ws_bytes = bytes;
  return RTAT_STATUS_SUCCESS;
}

size_t rtat_dtrsm_workspace_bytes(rtat_side_t side, int m, int n) {
  return trsm_workspace_bytes(side == RTAT_SIDE_LEFT ? m : n);
}

rtat_status_t rtat_dgemm_ex(rtat_handle_t h, rtat_operation_t transa, rtat_operation_t transb,
                            int m, int n, int k, const double* alpha, const double* A, int lda,
                            const double* B, int ldb, const double* beta, double* C, int ldc,
                            int variant) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_op(transa) || !valid_op(transb)) return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr || beta == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_dgemm(h, transa == RTAT_OP_T, transb == RTAT_OP_T, m, n, k, *alpha, A, lda, B,
                      ldb, *beta, C, ldc, 0, variant);
}

rtat_status_t rtat_dgemm(rtat_handle_t h, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, int k, const double* alpha, const double* A, int lda,
                         const double* B, int ldb, const double* beta, double* C, int ldc) {
  return rtat_dgemm_ex(h, transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
                       RTAT_GEMM_AUTO);
}

rtat_status_t rtat_dsyrk_ex(rtat_handle_t h, rtat_fill_t uplo, rtat_operation_t trans, int n,
                            int k, const double* alpha, const double* A, int lda,
                            const double* beta, double* C, int ldc, int variant) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_fill(uplo) || !valid_op(trans)) return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr || beta == nullptr) return RTAT_STATUS_INVALID_VALUE;
  // op(A) op(A)^T: trans == N -> A (n x k) times A^T; trans == T -> A^T times A (A is k x n).
  const bool t = trans == RTAT_OP_T;
  return launch_dgemm(h, t, !t, n, n, k, *alpha, A, lda, A, lda, *beta, C, ldc,
                      uplo == RTAT_FILL_LOWER ? 1 : 2, variant);
}

rtat_status_t rtat_dsyrk(rtat_handle_t h, rtat_fill_t uplo, rtat_operation_t trans, int n, int k,
                         const double* alpha, const double* A, int lda, const double* beta,
                         double* C, int ldc) {
  return rtat_dsyrk_ex(h, uplo, trans, n, k, alpha, A, lda, beta, C, ldc, RTAT_GEMM_AUTO);
}

rtat_status_t rtat_dtrsm_ex(rtat_handle_t h, rtat_side_t side, rtat_fill_t uplo,
                            rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                            const double* alpha, const double* A, int lda, double* B, int ldb,
                            int variant) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_side(side) || !valid_fill(uplo) || !valid_op(trans) || !valid_diag(diag))
    return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_trsm<double>(h, side == RTAT_SIDE_LEFT, uplo == RTAT_FILL_LOWER, trans == RTAT_OP_T,
                      diag == RTAT_DIAG_UNIT, m, n, *alpha, A, lda, B, ldb, variant);
}

rtat_status_t rtat_dtrsm(rtat_handle_t h, rtat_side_t side, rtat_fill_t uplo,
                         rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                         const double* alpha, const double* A, int lda, double* B, int ldb) {
  return rtat_dtrsm_ex(h, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, RTAT_GEMM_AUTO);
}

rtat_status_t rtat_dtrsm_static(rtat_handle_t h, rtat_side_t side, rtat_fill_t uplo,
                                rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                                const double* alpha, const double* A, int lda, double* B,
                                int ldb) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_side(side) || !valid_fill(uplo) || !valid_op(trans) || !valid_diag(diag))
    return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr) return RTAT_STATUS_INVALID_VALUE;
  const int na = side == RTAT_SIDE_LEFT ? m : n;
  if (na > RTAT_DTRSM_STATIC_MAX_ORDER) return RTAT_STATUS_NOT_SUPPORTED;
  if (h->static_ws == nullptr) return RTAT_STATUS_NOT_INITIALIZED;
  // The solve runs as it does with a lent workspace (no allocation anywhere below, GEMM
  // tails unsplit), the lent buffer being this device's static array.  Every element of
  // the scratch a solve reads, it has written first: nothing needs clearing between calls.
  void* const lent = h->user_ws;
  const size_t lent_bytes = h->user_ws_bytes;
  h->user_ws = h->static_ws;
  h->user_ws_bytes = STATIC_SCRATCH_BYTES;
  const rtat_status_t st =
      launch_trsm<double>(h, side == RTAT_SIDE_LEFT, uplo == RTAT_FILL_LOWER, trans == RTAT_OP_T,
                          diag == RTAT_DIAG_UNIT, m, n, *alpha, A, lda, B, ldb, RTAT_GEMM_AUTO);
  h->user_ws = lent;
  h->user_ws_bytes = lent_bytes;
  return st;
}

rtat_status_t rtat_dgeam(rtat_handle_t h, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, const double* alpha, const double* A, int lda,
                         const double* beta, const double* B, int ldb, double* C, int ldc) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_op(transa) || !valid_op(transb)) return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr || beta == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_geam<double>(h, transa == RTAT_OP_T, transb == RTAT_OP_T, m, n, *alpha, A, lda,
                             *beta, B, ldb, C, ldc);
}

rtat_status_t rtat_sgemm_ex(rtat_handle_t h, rtat_operation_t transa, rtat_operation_t transb,
                            int m, int n, int k, const float* alpha, const float* A, int lda,
                            const float* B, int ldb, const float* beta, float* C, int ldc,
                            int variant) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_op(transa) || !valid_op(transb)) return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr || beta == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_gemm<float>(h, transa == RTAT_OP_T, transb == RTAT_OP_T, m, n, k, *alpha, A, lda,
                            B, ldb, *beta, C, ldc, 0, variant);
}

rtat_status_t rtat_sgemm(rtat_handle_t h, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, int k, const float* alpha, const float* A, int lda,
                         const float* B, int ldb, const float* beta, float* C, int ldc) {
  return rtat_sgemm_ex(h, transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
                       RTAT_GEMM_AUTO);
}

rtat_status_t rtat_ssyrk_ex(rtat_handle_t h, rtat_fill_t uplo, rtat_operation_t trans, int n,
                            int k, const float* alpha, const float* A, int lda,
                            const float* beta, float* C, int ldc, int variant) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_fill(uplo) || !valid_op(trans)) return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr || beta == nullptr) return RTAT_STATUS_INVALID_VALUE;
  const bool t = trans == RTAT_OP_T;
  return launch_gemm<float>(h, t, !t, n, n, k, *alpha, A, lda, A, lda, *beta, C, ldc,
                            uplo == RTAT_FILL_LOWER ? 1 : 2, variant);
}

rtat_status_t rtat_ssyrk(rtat_handle_t h, rtat_fill_t uplo, rtat_operation_t trans, int n, int k,
                         const float* alpha, const float* A, int lda, const float* beta,
                         float* C, int ldc) {
  return rtat_ssyrk_ex(h, uplo, trans, n, k, alpha, A, lda, beta, C, ldc, RTAT_GEMM_AUTO);
}

rtat_status_t rtat_strsm_ex(rtat_handle_t h, rtat_side_t side, rtat_fill_t uplo,
                            rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                            const float* alpha, const float* A, int lda, float* B, int ldb,
                            int variant) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_side(side) || !valid_fill(uplo) || !valid_op(trans) || !valid_diag(diag))
    return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_trsm<float>(h, side == RTAT_SIDE_LEFT, uplo == RTAT_FILL_LOWER,
                            trans == RTAT_OP_T, diag == RTAT_DIAG_UNIT, m, n, *alpha, A, lda, B,
                            ldb, variant);
}

rtat_status_t rtat_strsm(rtat_handle_t h, rtat_side_t side, rtat_fill_t uplo,
                         rtat_operation_t trans, rtat_diag_t diag, int m, int n,
                         const float* alpha, const float* A, int lda, float* B, int ldb) {
  return rtat_strsm_ex(h, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, RTAT_GEMM_AUTO);
}

rtat_status_t rtat_sgeam(rtat_handle_t h, rtat_operation_t transa, rtat_operation_t transb,
                         int m, int n, const float* alpha, const float* A, int lda,
                         const float* beta, const float* B, int ldb, float* C, int ldc) {
  RTAT_CHECK_HANDLE(h);
  if (!valid_op(transa) || !valid_op(transb)) return RTAT_STATUS_INVALID_ENUM;
  if (alpha == nullptr || beta == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_geam<float>(h, transa == RTAT_OP_T, transb == RTAT_OP_T, m, n, *alpha, A, lda,
                            *beta, B, ldb, C, ldc);
}

const char* rtat_gemm_variant_name(int variant) {
  switch (variant) {
    case RTAT_GEMM_AUTO: return "auto";
    case RTAT_GEMM_T256x128: return "256x128";
    case RTAT_GEMM_T128x128: return "128x128";
    case RTAT_GEMM_T128x64: return "128x64";
    case RTAT_GEMM_T64x64: return "64x64";
    default: return nullptr;
  }
}

const char* rtat_tail_mode_name(int mode) {
  switch (mode) {
    case RTAT_TAIL_AUTO: return "auto";
    case RTAT_TAIL_WHOLE: return "whole";
    case RTAT_TAIL_SPLIT: return "split";
    default: return nullptr;
  }
}

const char* rtat_trsm_panel_name(int panel) {
  switch (panel) {
    case RTAT_PANEL_AUTO: return "auto";
    case RTAT_PANEL_512: return "512";
    case RTAT_PANEL_1024: return "1024";
    default: return nullptr;
  }
}

rtat_status_t rtat_last_launch(rtat_handle_t h, rtat_launch_info_t* info) {
  RTAT_CHECK_HANDLE(h);
  if (info == nullptr) return RTAT_STATUS_INVALID_VALUE;
  *info = h->last;
  if (h->last_bm > 0) snprintf(info->tile, sizeof(info->tile), "%dx%d", h->last_bm, h->last_bn);
  return RTAT_STATUS_SUCCESS;
}

rtat_status_t rtat_dfill(rtat_handle_t h, double* A, int m, int n, int ld, uint64_t seed,
                         int kind) {
  RTAT_CHECK_HANDLE(h);
  return launch_fill<double>(h, A, m, n, ld, seed, kind);
}

rtat_status_t rtat_sfill(rtat_handle_t h, float* A, int m, int n, int ld, uint64_t seed,
                         int kind) {
  RTAT_CHECK_HANDLE(h);
  return launch_fill<float>(h, A, m, n, ld, seed, kind);
}

rtat_status_t rtat_device_peaks(rtat_handle_t h, double* fp64_mfma_flops,
                                double* hbm_bytes_per_s, int* compute_units) {
  RTAT_CHECK_HANDLE(h);
  // 128 fp64 matrix flop per clock per CU on CDNA4 (v_mfma_f64_16x16x4: 2048 flop in 64
  // cycles on each of 4 SIMDs).
  if (fp64_mfma_flops) *fp64_mfma_flops = (double)h->compute_units * h->clock_hz * 128.0;
  if (hbm_bytes_per_s) *hbm_bytes_per_s = h->mem_bytes_per_s;
  if (compute_units) *compute_units = h->compute_units;
  return RTAT_STATUS_SUCCESS;
}

rtat_status_t rtat_dmove_pair(rtat_handle_t h, const rtat_move_t* first,
                              const rtat_move_t* second) {
  RTAT_CHECK_HANDLE(h);
  if (first == nullptr || second == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_move_pair<double>(h, first, second);
}

rtat_status_t rtat_smove_pair(rtat_handle_t h, const rtat_move_t* first,
                              const rtat_move_t* second) {
  RTAT_CHECK_HANDLE(h);
  if (first == nullptr || second == nullptr) return RTAT_STATUS_INVALID_VALUE;
  return launch_move_pair<float>(h, first, second);
}

rtat_status_t rtat_hbm_probe(rtat_handle_t h, int kind, const void* src, void* dst,
                             size_t bytes) {
  RTAT_CHECK_HANDLE(h);
  return launch_probe(h, kind, src, dst, bytes);
}

const char* rtat_version(void) { return "rtat-native 0.1 gfx950"; }

}  // extern "C"
