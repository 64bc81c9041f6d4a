// A snapshot of every timing an executor has recorded: per problem key and variant the raw
// samples, their count and mean, flop rates, and the JSON report run_tests prints (reference
// src/planning/planner_statistics.h).
#pragma once
#include <json_encoding.h>

#include <map>
#include <numeric>
#include <vector>

template <typename Key, typename Opts>
class Planner_Statistics {
 public:
  template <typename V>
  using Per_Variant = std::map<Key, std::map<Opts, V>>;
  using Samples = std::vector<float>;  // milliseconds

  Planner_Statistics(Per_Variant<Samples> recorded) : times(std::move(recorded)) {
    each([&](const Key& key, const Opts& opt, const Samples& ms) {
      counts[key][opt] = ms.size();
      const double sum = std::accumulate(ms.begin(), ms.end(), 0.0);
      means[key][opt] = ms.empty() ? 0.f : (float)(sum / (double)ms.size());
    });
  }

  const Per_Variant<Samples>& get_times() { return times; }
  const Per_Variant<float>& get_means() { return means; }
  const Per_Variant<size_t>& get_counts() { return counts; }

  // flop/s of every sample, for keys that define flopcount().  (The reference declares this
  // with a mismatched return type and none of its keys has flopcount(),
  // planner_statistics.h:35-48; here it works.)
  Per_Variant<std::vector<double>> get_floprates() {
    Per_Variant<std::vector<double>> rates;
    each([&](const Key& key, const Opts& opt, const Samples& ms) {
      for (float t : ms) rates[key][opt].push_back(key.flopcount() / (t * 1e-3));
    });
    return rates;
  }

  // [{"key": <key>, "options": [{"option": <variant>, "times": [ms, ...]}, ...]}, ...]
  rtat::Json json() {
    rtat::Json report = rtat::Json::array();
    for (auto& [key, variants] : times) {
      rtat::Json options = rtat::Json::array();
      for (auto& [opt, ms] : variants) {
        rtat::Json o;
        o["option"] = to_json(opt);
        o["times"] = rtat::Json(ms);
        options.push_back(o);
      }
      rtat::Json entry;
      entry["key"] = to_json(key);
      entry["options"] = options;
      report.push_back(entry);
    }
    return report;
  }

 private:
  template <typename Visit>
  void each(Visit&& visit) {
    for (auto& [key, variants] : times)
      for (auto& [opt, ms] : variants) visit(key, opt, ms);
  }

  Per_Variant<Samples> times;
  Per_Variant<float> means;
  Per_Variant<size_t> counts;
};
