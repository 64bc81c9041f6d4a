// Times work enqueued on one stream by bracketing it with two events (reference
// src/timing/device_timer.h, device_timer.cpp).
#pragma once
#include <gpu-api.h>

#include <optional>

namespace rtat {

class Device_Timer {
 public:
  // ASYNCHRONOUS: bracket the work and return.  SEMI_SYNCHRONOUS: drain the device first, so
  // that earlier work cannot bleed into the interval.  SYNCHRONOUS: also wait for the work to
  // finish before returning.  (reference device_timer.h:10-31)
  enum Mode { ASYNCHRONOUS = 0, SEMI_SYNCHRONOUS = 1, SYNCHRONOUS = 2 };

  template <typename Func>
  Device_Timer(Func&& work, Stream s, Mode mode = ASYNCHRONOUS) : bracket(Bracket{}) {
    if (mode != ASYNCHRONOUS) gpuAssert(gpu::DeviceSynchronize());
    bracket->opening.record(s);
    work(s);
    bracket->closing.record(s);
    if (mode == SYNCHRONOUS) bracket->closing.synchronize();
  }

  // A timer that already knows its result (measurements made elsewhere, tests).
  explicit Device_Timer(float known_ms) : ms(known_ms) {}

  Device_Timer(Device_Timer&&) = default;
  Device_Timer& operator=(Device_Timer&&) = default;

  // Elapsed milliseconds if the work has finished, nothing otherwise; never blocks.  The
  // events are given back to the runtime as soon as the time has been read.
  std::optional<float> query_time() {
    if (!bracket) return ms;
    if (!bracket->opening.query() || !bracket->closing.query()) return std::nullopt;
    ms = Event::elapsed_time(bracket->opening, bracket->closing);
    bracket.reset();
    return ms;
  }

  // Elapsed milliseconds, waiting for the work to finish first.
  float time() {
    if (bracket) bracket->closing.synchronize();
    return *query_time();
  }

 private:
  struct Bracket {
    Event opening, closing;
  };
  std::optional<Bracket> bracket;  // empty once the time is known
  float ms = -1.0f;
};

}  // namespace rtat
