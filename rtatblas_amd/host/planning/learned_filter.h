// An Option_Filter learned from timings: for a class of problems it admits only the variants
// that came close to the fastest on some problem of that class already measured, so that the
// planner's exploration of a new problem skips variants that never paid off for its kind.
// (No counterpart in the reference, which only has the hand-written filter hook,
// planning_system.h:14-35.)
#pragma once
#include <algorithm>
#include <cmath>
#include <limits>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "planning_system.h"

namespace rtat {

// Problem classes: the flags of the key plus the power of two nearest to the cube root of
// its flop count, so that problems of similar size and identical flags share what was learned.
inline std::string size_bucket(double flops) {
  const double edge = std::cbrt(flops > 1.0 ? flops : 1.0);
  return std::to_string((int)std::lround(std::log2(edge)));
}
inline std::string shape_class(const GEMM_Key& k) {
  return std::string(k.transa) + std::string(k.transb) + "/" + size_bucket(k.flopcount());
}
inline std::string shape_class(const SYRK_Key& k) {
  return std::string(k.uplo) + std::string(k.trans) + "/" + size_bucket(k.flopcount());
}
inline std::string shape_class(const TRSM_Key& k) {
  return std::string(k.side) + std::string(k.uplo) + std::string(k.trans) + std::string(k.diag) +
         "/" + size_bucket(k.flopcount());
}

// Learns from `stats` (any Planner_Statistics of the same key and variant types).  A variant
// is kept for a class when its median time on some problem of the class is within
// (1 + slack) of that problem's fastest median.  The default variant is always admitted (the
// planner falls back to it when scratch is short), and a class nothing is known about admits
// every variant.
template <typename Key, typename Opts>
Option_Filter<Key, Opts> learn_filter(Planner_Statistics<Key, Opts>& stats, float slack = 0.1f) {
  auto median = [](std::vector<float> ms) {
    std::sort(ms.begin(), ms.end());
    return ms[ms.size() / 2];
  };
  auto kept = std::make_shared<std::map<std::string, std::set<std::string>>>();
  for (auto& [key, variants] : stats.get_times()) {
    float best = std::numeric_limits<float>::max();
    for (auto& [opt, ms] : variants)
      if (!ms.empty()) best = std::min(best, median(ms));
    std::set<std::string>& names = (*kept)[shape_class(key)];
    for (auto& [opt, ms] : variants)
      if (!ms.empty() && median(ms) <= best * (1.0f + slack)) names.insert(std::string(opt));
  }
  const std::string fallback = std::string(Opts::default_opts());
  return Option_Filter<Key, Opts>([kept, fallback](std::pair<Opts, Key> candidate) {
    const std::string name = std::string(candidate.first);
    if (name == fallback) return true;
    auto cls = kept->find(shape_class(candidate.second));
    return cls == kept->end() || cls->second.count(name) != 0;
  });
}

}  // namespace rtat
