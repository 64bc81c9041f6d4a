#include "timer_bank.h"

#include <algorithm>
#include <cmath>
#include <numeric>

namespace rtat {

void Timer_Bank::harvest() {
  while (!pending.empty()) {
    auto t = pending.front().query_time();
    if (!t) break;  // in stream order: nothing behind an unfinished timer can be done
    times.push_back(*t);
    pending.pop_front();
  }
}

void Timer_Bank::append(Device_Timer& timer) { pending.push_back(std::move(timer)); }
void Timer_Bank::append(Device_Timer&& timer) { pending.push_back(std::move(timer)); }

void Timer_Bank::synchronize() {
  for (; !pending.empty(); pending.pop_front()) times.push_back(pending.front().time());
}

size_t Timer_Bank::size() const { return pending.size() + times.size(); }

size_t Timer_Bank::completed() {
  harvest();
  return times.size();
}

const std::vector<float>& Timer_Bank::get_times() {
  harvest();
  return times;
}

float Timer_Bank::mean() {
  if (times.empty()) return NAN;
  return (float)(std::accumulate(times.begin(), times.end(), 0.0) / (double)times.size());
}

float Timer_Bank::median() {
  if (times.empty()) return NAN;
  std::vector<float> s(times);
  std::sort(s.begin(), s.end());
  return s[s.size() / 2];
}

float Timer_Bank::minimum() {
  if (times.empty()) return NAN;
  return *std::min_element(times.begin(), times.end());
}

}  // namespace rtat
