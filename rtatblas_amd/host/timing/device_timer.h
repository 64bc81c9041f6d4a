// Event-pair timer around work enqueued on one stream (reference src/timing/device_timer.h).
#pragma once
#include <gpu-api.h>

#include <optional>

namespace rtat {

class Device_Timer {
 public:
  // ASYNCHRONOUS: just bracket the work with events.  SEMI_SYNCHRONOUS: drain the device
  // first so earlier work cannot bleed into the interval.  SYNCHRONOUS: also wait for the
  // end event before returning.  (reference device_timer.h:10-31)
  enum Mode { ASYNCHRONOUS = 0, SEMI_SYNCHRONOUS = 1, SYNCHRONOUS = 2 };

  template <typename Func>
  Device_Timer(Func&& work, Stream s, Mode mode = ASYNCHRONOUS)
      : start(std::make_unique<Event>()), end(std::make_unique<Event>()) {
    if (mode != ASYNCHRONOUS) gpuAssert(gpu::DeviceSynchronize());
    start->record(s);
    work(s);
    end->record(s);
    if (mode == SYNCHRONOUS) end->synchronize();
  }

  // A timer that already knows its result (measurements made elsewhere, tests).
  explicit Device_Timer(float known_ms) : elapsed(known_ms) {}

  Device_Timer(Device_Timer&&) = default;
  Device_Timer& operator=(Device_Timer&&) = default;

  // Elapsed ms if both events have completed, nothing otherwise; never blocks.
  std::optional<float> query_time();
  // Elapsed ms, blocking until the end event has completed.
  float time();

 private:
  std::unique_ptr<Event> start, end;  // released once the time has been read
  float elapsed = -1.0f;
};

}  // namespace rtat
