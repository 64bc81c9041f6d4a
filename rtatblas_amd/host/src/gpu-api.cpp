#include "gpu-api.h"

namespace rtat {

namespace gpu {
const char* blasGetStatusString(blasStatus_t s) {
  switch (s) {
    case RTAT_STATUS_SUCCESS: return "success";
    case RTAT_STATUS_NOT_INITIALIZED: return "not initialized";
    case RTAT_STATUS_ALLOC_FAILED: return "allocation failed";
    case RTAT_STATUS_INVALID_VALUE: return "invalid value";
    case RTAT_STATUS_EXECUTION_FAILED: return "kernel launch failed";
    case RTAT_STATUS_NOT_SUPPORTED: return "not supported";
    case RTAT_STATUS_HANDLE_IS_NULLPTR: return "null handle";
    case RTAT_STATUS_INVALID_ENUM: return "invalid enum";
  }
  return "unknown status";
}
}  // namespace gpu

// An owning handle's deleter destroys the resource; a wrapping handle's deleter does nothing.
Stream::Stream() {
  gpu::Stream_t s = nullptr;
  gpuAssert(gpu::StreamCreate(&s));
  raw.reset(s, [](gpu::Stream_t p) { gpuAssert(gpu::StreamDestroy(p)); });
}
Stream::Stream(gpu::Stream_t stream) : raw(stream, [](gpu::Stream_t) {}) {}
void Stream::wait_event(Event e) { gpuAssert(gpu::StreamWaitEvent(*this, e, 0)); }
void Stream::synchronize() { gpuAssert(gpu::StreamSynchronize(*this)); }

Event::Event() {
  gpu::Event_t e = nullptr;
  gpuAssert(gpu::EventCreate(&e));
  raw.reset(e, [](gpu::Event_t p) { gpuAssert(gpu::EventDestroy(p)); });
}
Event::Event(gpu::Event_t event) : raw(event, [](gpu::Event_t) {}) {}
void Event::record(Stream s) { gpuAssert(gpu::EventRecord(*this, s)); }
void Event::synchronize() { gpuAssert(gpu::EventSynchronize(*this)); }
bool Event::query() { return gpu::EventQuery(*this) == gpu::Success; }
float Event::elapsed_time(Event start, Event end) {
  float ms = 0.f;
  return gpu::EventElapsedTime(&ms, start, end) == gpu::Success ? ms : NAN;
}

Device_RNG::Device_RNG() : state(std::make_shared<State>()) {
  blas_check(rtat_create(&state->handle), "rtat_create (Device_RNG)");
}
Device_RNG::State::~State() {
  if (handle) rtat_destroy(handle);
}
void Device_RNG::set_stream(Stream s) {
  blas_check(rtat_set_stream(state->handle, static_cast<gpu::Stream_t>(s)), "rtat_set_stream");
}

namespace {
// A flat run of `len` elements is filled as a matrix of at most 2^20 rows per column.
template <typename T, typename Fill>
void fill_flat(rtat_handle_t h, T* A, size_t len, uint64_t seed, Fill fill) {
  constexpr size_t ROWS = size_t(1) << 20;
  const size_t full_cols = len / ROWS, tail = len % ROWS;
  size_t done_cols = 0;
  while (done_cols < full_cols) {
    const size_t cols = std::min<size_t>(full_cols - done_cols, 1024);
    blas_check(fill(h, A + done_cols * ROWS, (int)ROWS, (int)cols, (int)ROWS,
                    seed + 0x9E3779B9ull * (done_cols + 1), RTAT_FILL_UNIT_INTERVAL),
               "rtat_fill");
    done_cols += cols;
  }
  if (tail)
    blas_check(fill(h, A + full_cols * ROWS, (int)tail, 1, (int)tail, seed ^ 0xabcdef,
                    RTAT_FILL_UNIT_INTERVAL),
               "rtat_fill");
}
}  // namespace

template <>
void Device_RNG::uniform<double>(double* A, size_t len) {
  fill_flat(state->handle, A, len, state->next++, rtat_dfill);
}
template <>
void Device_RNG::uniform<float>(float* A, size_t len) {
  fill_flat(state->handle, A, len, state->next++, rtat_sfill);
}

}  // namespace rtat
