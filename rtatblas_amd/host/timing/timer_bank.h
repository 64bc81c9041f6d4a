// FIFO of in-flight timers plus the times already harvested (reference src/timing/timer_bank.h).
#pragma once
#include <deque>
#include <vector>

#include "device_timer.h"

namespace rtat {

class Timer_Bank {
 public:
  void append(Device_Timer& timer);   // takes the timer over (the argument is moved from)
  void append(Device_Timer&& timer);
  const std::vector<float>& get_times();  // harvests whatever has completed, never blocks
  void synchronize();                     // blocks until every pending timer is harvested
  size_t size() const;                    // pending + harvested
  size_t completed();                     // harvested, after a non-blocking harvest

  // Order statistics over the harvested times (after synchronize()); NaN when empty.
  float mean();
  float median();
  float minimum();

 private:
  void harvest();
  std::deque<Device_Timer> pending;
  std::vector<float> times;
};

}  // namespace rtat
