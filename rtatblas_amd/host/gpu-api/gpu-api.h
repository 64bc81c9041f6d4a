// rtat::gpu — the device API the upper layers are written against.
//
// Same names as the reference's src/gpu-api/gpu-api.h (runtime calls :44-85, BLAS calls
// :87-113, RNG :115-121, RAII wrappers :157-241, string-backed enums :246-325), but nothing
// here forwards to a vendor BLAS: the BLAS half binds to the gfx950 kernels behind the C ABI
// in rtat_native.h, the runtime half is plain HIP, and random fills come from the library's
// own counter-based generator.  There is one back end; no build-time switch.
#pragma once
#include <hip/hip_runtime_api.h>

#include <array>
#include <cmath>
#include <iostream>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>

#include "rtat_native.h"

namespace rtat {

namespace gpu {
// ---- runtime (reference gpu-api.h:44-85) ------------------------------------------------
using Error_t = hipError_t;
using Stream_t = hipStream_t;
using Event_t = hipEvent_t;
constexpr Error_t Success = hipSuccess;
constexpr Error_t ErrorInvalidResourceHandle = hipErrorInvalidResourceHandle;

inline Error_t SetDevice(int d) { return hipSetDevice(d); }
inline Error_t GetDevice(int* d) { return hipGetDevice(d); }
inline Error_t GetDeviceCount(int* n) { return hipGetDeviceCount(n); }
inline Error_t DeviceSynchronize() { return hipDeviceSynchronize(); }
inline Error_t MemGetInfo(size_t* free_b, size_t* total_b) { return hipMemGetInfo(free_b, total_b); }
inline const char* GetErrorString(Error_t e) { return hipGetErrorString(e); }

template <typename T>
inline Error_t Malloc(T** ptr, size_t bytes) { return hipMalloc(reinterpret_cast<void**>(ptr), bytes); }
inline Error_t Free(void* ptr) { return hipFree(ptr); }

constexpr hipMemcpyKind MemcpyDeviceToDevice = hipMemcpyDeviceToDevice;
constexpr hipMemcpyKind MemcpyDeviceToHost = hipMemcpyDeviceToHost;
constexpr hipMemcpyKind MemcpyHostToDevice = hipMemcpyHostToDevice;
inline Error_t Memcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind) {
  return hipMemcpy(dst, src, bytes, kind);
}
inline Error_t MemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind kind,
                           Stream_t s) {
  return hipMemcpyAsync(dst, src, bytes, kind, s);
}
inline Error_t Memset(void* dst, int value, size_t bytes) { return hipMemset(dst, value, bytes); }

inline Error_t StreamCreate(Stream_t* s) { return hipStreamCreate(s); }
inline Error_t StreamDestroy(Stream_t s) { return hipStreamDestroy(s); }
inline Error_t StreamSynchronize(Stream_t s) { return hipStreamSynchronize(s); }
inline Error_t StreamWaitEvent(Stream_t s, Event_t e, unsigned flags) {
  return hipStreamWaitEvent(s, e, flags);
}
inline Error_t EventCreate(Event_t* e) { return hipEventCreate(e); }
inline Error_t EventDestroy(Event_t e) { return hipEventDestroy(e); }
inline Error_t EventRecord(Event_t e, Stream_t s) { return hipEventRecord(e, s); }
inline Error_t EventSynchronize(Event_t e) { return hipEventSynchronize(e); }
inline Error_t EventQuery(Event_t e) { return hipEventQuery(e); }
inline Error_t EventElapsedTime(float* ms, Event_t a, Event_t b) {
  return hipEventElapsedTime(ms, a, b);
}

// ---- BLAS (reference gpu-api.h:87-113): the native C ABI under the reference's names ---
using blasHandle_t = rtat_handle_t;
using blasStatus_t = rtat_status_t;
using blasOperation_t = rtat_operation_t;
using blasFillMode_t = rtat_fill_t;
using blasSideMode_t = rtat_side_t;
using blasDiagType_t = rtat_diag_t;
constexpr blasStatus_t BLAS_STATUS_SUCCESS = RTAT_STATUS_SUCCESS;
constexpr blasOperation_t BLAS_OP_N = RTAT_OP_N;
constexpr blasOperation_t BLAS_OP_T = RTAT_OP_T;
constexpr blasFillMode_t BLAS_FILL_MODE_UPPER = RTAT_FILL_UPPER;
constexpr blasFillMode_t BLAS_FILL_MODE_LOWER = RTAT_FILL_LOWER;
constexpr blasSideMode_t BLAS_SIDE_LEFT = RTAT_SIDE_LEFT;
constexpr blasSideMode_t BLAS_SIDE_RIGHT = RTAT_SIDE_RIGHT;
constexpr blasDiagType_t BLAS_DIAG_NON_UNIT = RTAT_DIAG_NON_UNIT;
constexpr blasDiagType_t BLAS_DIAG_UNIT = RTAT_DIAG_UNIT;

constexpr auto blasCreate = rtat_create;
constexpr auto blasDestroy = rtat_destroy;
inline blasStatus_t blasSetStream(blasHandle_t h, Stream_t s) { return rtat_set_stream(h, s); }
inline blasStatus_t blasGetStream(blasHandle_t h, Stream_t* s) {
  rtat_stream_t raw = nullptr;
  blasStatus_t st = rtat_get_stream(h, &raw);
  *s = static_cast<Stream_t>(raw);
  return st;
}
constexpr auto blasDgemm = rtat_dgemm;
constexpr auto blasDsyrk = rtat_dsyrk;
constexpr auto blasDtrsm = rtat_dtrsm;
constexpr auto blasDgeam = rtat_dgeam;
constexpr auto blasSgemm = rtat_sgemm;
constexpr auto blasSsyrk = rtat_ssyrk;
constexpr auto blasStrsm = rtat_strsm;
constexpr auto blasSgeam = rtat_sgeam;
// Kernel-variant entry points (no counterpart in the reference).
constexpr auto blasDgemmEx = rtat_dgemm_ex;
constexpr auto blasDsyrkEx = rtat_dsyrk_ex;
constexpr auto blasDtrsmEx = rtat_dtrsm_ex;
constexpr auto blasSgemmEx = rtat_sgemm_ex;
constexpr auto blasSsyrkEx = rtat_ssyrk_ex;
constexpr auto blasStrsmEx = rtat_strsm_ex;
// Two moves (copy / pad copy / transpose) in one launch.
using blasMove_t = rtat_move_t;
constexpr auto blasDmovePair = rtat_dmove_pair;
constexpr auto blasSmovePair = rtat_smove_pair;

const char* blasGetStatusString(blasStatus_t s);
}  // namespace gpu

// Reference gpu-api.h:128-138: report a failed runtime call on stderr and carry on.
#define gpuAssert(ans) \
  { ::rtat::gpu_error_check((ans), __FILE__, __LINE__); }

inline void gpu_error_check(gpu::Error_t code, const char* file, int line) {
  if (code != gpu::Success)
    std::cerr << "GPU Error: " << gpu::GetErrorString(code) << " " << file << " " << line
              << std::endl;
}

// Unlike the reference, which drops every BLAS status (e.g. matrixop.h:302,340,391), the
// matrix-op nodes route theirs through here: a failed launch throws.
inline void blas_check(gpu::blasStatus_t st, const char* what) {
  if (st != gpu::BLAS_STATUS_SUCCESS)
    throw std::runtime_error(std::string(what) + " failed: " + gpu::blasGetStatusString(st));
}

class Event;

// Copyable handle on a stream; the last copy of an owning handle destroys the stream
// (reference gpu-api.h:157-176, gpu-api.cpp:19-56).
class Stream {
 public:
  Stream();                       // creates and owns a new stream
  Stream(gpu::Stream_t stream);   // wraps an existing stream, never destroys it
  operator gpu::Stream_t() const { return raw.get(); }
  void wait_event(Event e);
  void synchronize();

 private:
  std::shared_ptr<std::remove_pointer_t<gpu::Stream_t>> raw;
};

// Copyable handle on an event (reference gpu-api.h:189-206, gpu-api.cpp:58-75).
class Event {
 public:
  Event();
  Event(gpu::Event_t event);
  operator gpu::Event_t() const { return raw.get(); }
  void record(Stream s);
  void synchronize();
  bool query();
  // Milliseconds between two recorded events; NaN when the runtime reports an error.
  static float elapsed_time(Event start, Event end);

 private:
  std::shared_ptr<std::remove_pointer_t<gpu::Event_t>> raw;
};

// Device-side operand filler (reference gpu-api.h:217-241 wraps a hipRAND generator).  Here:
// the library's counter-based generator; every call draws from a fresh sub-stream, values
// uniform in (0, 1] like hiprandGenerateUniform.  seed() makes a run reproducible, which the
// reference's never-seeded generator is not across library versions.
class Device_RNG {
 public:
  Device_RNG();
  Device_RNG(Stream s) : Device_RNG() { set_stream(s); }
  void set_stream(Stream s);
  void seed(uint64_t s) { state->next = s; }

  template <typename T>
  void uniform(T* A, size_t len);

 private:
  struct State {
    rtat_handle_t handle = nullptr;
    uint64_t next = 0x5eed;
    ~State();
  };
  std::shared_ptr<State> state;
};

// Enum value <-> string, for the plan-JSON vocabulary (reference gpu-api.h:246-297).
template <class Table>
class String_Rep {
  using T = typename Table::value_type;
  T val;

 public:
  String_Rep(T val) : val(val) {}
  String_Rep(const std::string& str) {
    for (const auto& e : Table::entries)
      if (str == e.second) {
        val = e.first;
        return;
      }
    throw std::runtime_error("Invalid string " + str + " passed to string rep");
  }
  String_Rep(const char* str) : String_Rep(std::string(str)) {}

  operator T() const { return val; }
  operator std::string() const {
    for (const auto& e : Table::entries)
      if (e.first == val) return e.second;
    throw std::runtime_error("Invalid string rep value");
  }
  // The other value of a two-valued enum.
  String_Rep operator!() const {
    static_assert(Table::entries.size() == 2, "operator! needs a binary String_Rep");
    return String_Rep(Table::entries[0].first == val ? Table::entries[1].first
                                                     : Table::entries[0].first);
  }
  bool operator==(T o) const { return val == o; }
  bool operator!=(T o) const { return val != o; }
  friend std::ostream& operator<<(std::ostream& os, const String_Rep& r) {
    return os << std::string(r);
  }
};

struct BLAS_Operation_Table {
  using value_type = gpu::blasOperation_t;
  static constexpr std::array<std::pair<value_type, const char*>, 2> entries{
      {{gpu::BLAS_OP_N, "N"}, {gpu::BLAS_OP_T, "T"}}};
};
struct BLAS_Fill_Mode_Table {
  using value_type = gpu::blasFillMode_t;
  static constexpr std::array<std::pair<value_type, const char*>, 2> entries{
      {{gpu::BLAS_FILL_MODE_LOWER, "Lower"}, {gpu::BLAS_FILL_MODE_UPPER, "Upper"}}};
};
struct BLAS_Side_Table {
  using value_type = gpu::blasSideMode_t;
  static constexpr std::array<std::pair<value_type, const char*>, 2> entries{
      {{gpu::BLAS_SIDE_LEFT, "Left"}, {gpu::BLAS_SIDE_RIGHT, "Right"}}};
};
struct BLAS_Diag_Table {
  using value_type = gpu::blasDiagType_t;
  static constexpr std::array<std::pair<value_type, const char*>, 2> entries{
      {{gpu::BLAS_DIAG_UNIT, "Unit"}, {gpu::BLAS_DIAG_NON_UNIT, "Non-Unit"}}};
};
using BLAS_Operation = String_Rep<BLAS_Operation_Table>;
using BLAS_Fill_Mode = String_Rep<BLAS_Fill_Mode_Table>;
using BLAS_Side = String_Rep<BLAS_Side_Table>;
using BLAS_Diag = String_Rep<BLAS_Diag_Table>;

}  // namespace rtat
