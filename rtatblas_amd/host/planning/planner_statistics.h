// Snapshot of every recorded timing, with counts, means and the JSON report (reference
// src/planning/planner_statistics.h).
#pragma once
#include <json_encoding.h>

#include <algorithm>
#include <map>
#include <numeric>
#include <vector>

template <typename Key, typename Opts>
class Planner_Statistics {
  using Table = std::map<Key, std::map<Opts, std::vector<float>>>;
  Table times;
  std::map<Key, std::map<Opts, float>> means;
  std::map<Key, std::map<Opts, size_t>> counts;

 public:
  Planner_Statistics(Table recorded) : times(std::move(recorded)) {
    for (auto& [key, per_opt] : times)
      for (auto& [opt, ts] : per_opt) {
        counts[key][opt] = ts.size();
        means[key][opt] =
            ts.empty() ? 0.f : (float)(std::accumulate(ts.begin(), ts.end(), 0.0) / ts.size());
      }
  }

  const Table& get_times() { return times; }
  const std::map<Key, std::map<Opts, float>>& get_means() { return means; }
  const std::map<Key, std::map<Opts, size_t>>& get_counts() { return counts; }

  // flop/s of every sample, for keys that define flopcount() (times are in ms).  The
  // reference declares this with a mismatched return type and no key implements
  // flopcount() there (planner_statistics.h:35-48); here it works.
  std::map<Key, std::map<Opts, std::vector<double>>> get_floprates() {
    std::map<Key, std::map<Opts, std::vector<double>>> rates;
    for (auto& [key, per_opt] : times)
      for (auto& [opt, ts] : per_opt)
        for (float ms : ts) rates[key][opt].push_back(key.flopcount() / (ms * 1e-3));
    return rates;
  }

  // [{"key": <key>, "options": [{"option": <variant>, "times": [ms, ...]}, ...]}, ...]
  rtat::Json json() {
    rtat::Json out = rtat::Json::array();
    for (auto& [key, per_opt] : times) {
      rtat::Json entry;
      entry["key"] = to_json(key);
      entry["options"] = rtat::Json::array();
      for (auto& [opt, ts] : per_opt) {
        rtat::Json o;
        o["option"] = to_json(opt);
        o["times"] = rtat::Json(ts);
        entry["options"].push_back(o);
      }
      out.push_back(entry);
    }
    return out;
  }
};
