#include "device_timer.h"

namespace rtat {

std::optional<float> Device_Timer::query_time() {
  if (elapsed >= 0.0f || !start) return elapsed;
  if (!start->query() || !end->query()) return std::nullopt;
  elapsed = Event::elapsed_time(*start, *end);
  start.reset();
  end.reset();
  return elapsed;
}

float Device_Timer::time() {
  if (start) {
    start->synchronize();
    end->synchronize();
  }
  return *query_time();
}

}  // namespace rtat
