// The autotuner: tries every admissible variant of a problem, then commits to the fastest
// (reference src/planning/planning_system.h).
#pragma once
#include <gemm.h>
#include <gpu-api.h>
#include <predicates.h>

#include <algorithm>
#include <limits>
#include <map>
#include <numeric>
#include <vector>

#include "planner_statistics.h"

namespace rtat {

// Which variants may be tried for which problem (reference planning_system.h:14-35).
template <typename Key, typename Opts>
class Option_Filter {
  Predicate<std::pair<Opts, Key>> admit;

 public:
  Option_Filter() : admit([](std::pair<Opts, Key>) { return true; }) {}
  Option_Filter(Predicate<std::pair<Opts, Key>> filter) : admit(filter) {}

  // Admitted variants in enumeration order.
  std::vector<Opts> apply(Key key) const {
    std::vector<Opts> kept;
    for (auto& opts : Opts::enumerate())
      if (admit(std::make_pair(opts, key))) kept.push_back(opts);
    return kept;
  }
};

template <typename Executor_Type>
class Planning_System {
 public:
  using Params = typename Executor_Type::Params_T;
  using Key = typename Executor_Type::Key_T;
  using Opts = typename Executor_Type::Opts_T;

  // How the samples of one variant are condensed into the figure variants are ranked by.
  // The reference ranks by the mean of (by default) a single sample; the median of a few is
  // robust against the one-off costs the first launch of a kernel carries (of an even number
  // the lower of the two middle ones: what disturbs a timing only ever adds to it).
  enum Statistic { MEAN, MEDIAN, MINIMUM };

 protected:
  Executor_Type executor;
  Option_Filter<Key, Opts> opt_filter;

  // A plan that does not fit the caller's workspace falls back to the variant that needs
  // none (reference :50-52).
  Opts degrade_plan(Params, Opts, Workspace) { return Opts::default_opts(); }

  size_t tests_until_converge = 3;
  Statistic statistic = MEDIAN;
  // Run-off: once every variant has its samples, those within refine_margin of the fastest
  // each get refine_tests more before the plan is committed.  With dozens of variants a few
  // percent apart, three samples each leave the fastest-looking one a likely outlier of a
  // slower variant (65536 x 256 x 256 through the 64 pad variants committed to a variant 4 %
  // slower than the plain call).  refine_tests = 0 commits at once, as the reference does.
  size_t refine_tests = 6;
  float refine_margin = 0.05f;
  // Commit rule: a variant counts as tied with the fastest when its figure is within
  // tie_margin of it, or within the spread of their own samples (the sum of the two variants'
  // distances from median to lower quartile: what separates them is then no more than their
  // noise - and the smallest of dozens of noisy figures is biased low to begin with).  Among tied variants the
  // plan goes to the default variant if it is one of them, otherwise to the one that needs the
  // least workspace (then the faster).  A bare argmin over figures a fraction of a percent
  // apart is a coin toss between them, and lands on a variant that first copies an operand
  // into hundreds of megabytes of scratch as readily as on the plain call.  0 restores the
  // bare argmin of the reference.
  // The spread widens the margin to at most twice tie_margin: a plan that ties with the fastest
  // may then be up to 0.5 % behind it by the figures, and the figure of the fastest of many is
  // the one biased low.  (With 0.5 % and no cap the default variant kept the plan where a
  // rival measured 0.55-0.63 % faster side by side.)
  float tie_margin = 0.0025f;
  // Bytes of workspace each variant asked for when it was last run (execute()): what the
  // commit rule compares, since create_plan sees a key, not the operands.
  std::map<Key, std::map<Opts, size_t>> workspace_seen;
  std::map<Key, Opts> converged_plans;
  Device_Timer::Mode sync_mode = Device_Timer::ASYNCHRONOUS;
  // Pseudo-random numbers for the order of the run-off; a fixed seed, so that the same
  // sequence of calls and timings gives the same plan.
  unsigned order_state = 0x9e3779b9u;
  unsigned draw() {
    order_state = order_state * 1664525u + 1013904223u;
    return order_state >> 8;
  }

  // How far a variant's samples scatter below their median: median - lower quartile (0 with
  // fewer than four samples).  Only the low side: what disturbs a timing only ever adds to it,
  // and the first samples of an exploration, taken while an idle GPU's clock still ramps,
  // would otherwise make every variant look as noisy as the ramp is long.
  static float spread_of(Timer_Bank& bank) {
    std::vector<float> ms = bank.get_times();
    if (ms.size() < 4) return 0.0f;
    std::sort(ms.begin(), ms.end());
    return ms[ms.size() / 2] - ms[ms.size() / 4];
  }

  // The figure a variant is ranked by.  Once the run-off has given a variant as many samples
  // as the exploration did, only the run-off's count.  The exploration picks who takes part;
  // fresh samples decide between them, which takes the selection bias out of the figures (the
  // variant that looked fastest among dozens did so partly by luck).  It also drops what the
  // exploration's neighbours did to a sample: a call right behind a kernel that left the GPU at
  // a lower clock measured 3-7 % slower (10007 x 4099 x 6151 behind any 64x64-tile variant),
  // and in passes over all variants the default variant always runs behind such a neighbour,
  // while in the run-off a variant runs among its peers.
  float figure_of(Timer_Bank& bank) {
    bank.synchronize();
    std::vector<float> ms = bank.get_times();
    if (refine_tests > 0 && ms.size() >= 2 * tests_until_converge)
      ms.erase(ms.begin(), ms.begin() + (long)tests_until_converge);
    if (ms.empty()) return std::numeric_limits<float>::quiet_NaN();
    switch (statistic) {
      case MEAN: return (float)(std::accumulate(ms.begin(), ms.end(), 0.0) / (double)ms.size());
      case MINIMUM: return *std::min_element(ms.begin(), ms.end());
      default:  // of an even number of samples the lower of the two in the middle
        std::sort(ms.begin(), ms.end());
        return ms[(ms.size() - 1) / 2];
    }
  }

 public:
  Planning_System() = default;
  Planning_System(Option_Filter<Key, Opts> opt_filter) : opt_filter(opt_filter) {}
  virtual ~Planning_System() = default;

  // The variant to run next for `key`: the committed one if there is one; otherwise the
  // admitted variant with the fewest samples so far while any has fewer than
  // tests_until_converge (passes over the variants in enumeration order, every second one
  // backwards); once all have enough, the one with the smallest figure or one tied with it,
  // which is then committed for good.  (reference :65-96, which with its single sample per
  // variant explores in the same order.  With several samples the passes are interleaved
  // rather than taken back to back, so that whatever drifts while the exploration runs — the
  // clock ramp of a GPU that was idle, above all — is spread over the variants instead of
  // charged to the first.)
  virtual Opts create_plan(Key key) {
    if (auto it = converged_plans.find(key); it != converged_plans.end()) return it->second;

    std::map<Opts, Timer_Bank>& timings = executor.get_timings(key);
    const auto candidates = opt_filter.apply(key);
    // The admitted variant with the fewest samples goes next.  Among several with as few, the
    // first in enumeration order when that count is even and the last when it is odd: the
    // passes over the variants alternate in direction, so that a variant is not always run
    // right behind the same neighbour.  What a variant leaves in the caches is felt by the
    // next one - with 65536 x 256 x 256 the first variant of every pass, the plain call, ran
    // right behind the variant that pads all three operands and measured 2 % slower than the
    // same launch further down the list, every time.
    // In the run-off (shuffled) any of those with as few, by a pseudo-random draw: there a
    // variant has few rivals, and with alternating passes it would only ever run behind the
    // same two of them.  If one of the two leaves the clock low, half of the variant's samples
    // are a percent or two high (10007 x 4099 x 6151, `128x128/auto`: 7.09 7.26 7.11 7.17 7.12 7.24
    // ms, pass by pass) and so is their median.
    auto fewest_sampled = [&](size_t limit, auto&& eligible, bool shuffled) -> const Opts* {
      const Opts* pick = nullptr;
      size_t fewest = limit, as_few = 0;
      for (size_t c = 0; c < candidates.size(); ++c) {
        if (!eligible(c)) continue;
        const size_t have = timings[candidates[c]].size();
        if (have < fewest) {
          fewest = have;
          pick = &candidates[c];
          as_few = 1;
        } else if (pick != nullptr && have == fewest) {
          ++as_few;
          if (shuffled ? draw() % as_few == 0 : (fewest & 1) != 0) pick = &candidates[c];
        }
      }
      return pick;
    };
    const Opts* next = fewest_sampled(tests_until_converge, [](size_t) { return true; }, false);
    if (next != nullptr) return *next;

    Opts best = Opts::default_opts();
    float best_time = std::numeric_limits<float>::max();
    std::vector<float> figures;
    figures.reserve(candidates.size());
    for (auto& opts : candidates) {
      const float t = figure_of(timings[opts]);
      figures.push_back(t);
      if (t < best_time) {
        best = opts;
        best_time = t;
      }
    }
    // Run-off among the variants close to the fastest: the one with the fewest samples goes
    // next until each of them has its extra samples.  The figures move as samples arrive, so
    // a variant may join or leave the group; no variant is ever sampled more than
    // tests_until_converge + refine_tests times, which bounds the exploration.
    // The default variant takes part when its fastest sample is that close: ties go to it
    // (below), so its figure has to be as good as its rivals', and its exploration samples are
    // the ones most likely to be off (the first call of all, and the neighbours named above).
    if (refine_tests > 0) {
      const size_t wanted = tests_until_converge + refine_tests;
      const float limit = best_time * (1.0f + refine_margin);
      const Opts plain = Opts::default_opts();
      auto is_close = [&](size_t c) {
        if (figures[c] <= limit) return true;
        if (candidates[c] < plain || plain < candidates[c]) return false;
        const std::vector<float>& ms = timings[candidates[c]].get_times();
        return !ms.empty() && *std::min_element(ms.begin(), ms.end()) <= limit;
      };
      size_t close = 0;
      for (size_t c = 0; c < candidates.size(); ++c)
        if (is_close(c)) ++close;
      next = fewest_sampled(wanted, is_close, true);
      if (close > 1 && next != nullptr) return *next;
    }
    // Ties go to the default variant, then to the smallest workspace.
    if (tie_margin > 0.0f) {
      const std::string plain = std::string(Opts::default_opts());
      const std::map<Opts, size_t>& asked = workspace_seen[key];
      auto bytes_of = [&](const Opts& o) {
        auto it = asked.find(o);
        return it == asked.end() ? std::numeric_limits<size_t>::max() : it->second;
      };
      size_t pick = candidates.size();
      const float best_spread = spread_of(timings[best]);
      for (size_t c = 0; c < candidates.size(); ++c) {
        const float noise = best_spread + spread_of(timings[candidates[c]]);
        const float slack = std::min(std::max(best_time * tie_margin, noise), 2.0f * best_time * tie_margin);
        if (figures[c] > best_time + slack) continue;
        if (std::string(candidates[c]) == plain) {
          pick = c;
          break;
        }
        if (pick == candidates.size() || bytes_of(candidates[c]) < bytes_of(candidates[pick]) ||
            (bytes_of(candidates[c]) == bytes_of(candidates[pick]) && figures[c] < figures[pick]))
          pick = c;
      }
      if (pick < candidates.size()) best = candidates[pick];
    }
    converged_plans.insert_or_assign(key, best);
    return best;
  }

  // Replace the filter that says which variants may be tried for which problem.  Plans already
  // committed stay as they are.
  void set_filter(Option_Filter<Key, Opts> filter) { opt_filter = std::move(filter); }
  // The variants create_plan considers for `key`, in enumeration order.
  std::vector<Opts> admitted(Key key) const { return opt_filter.apply(key); }
  // Variants within `margin` (a fraction) of the fastest count as tied with it; see tie_margin.
  void set_tie_margin(float margin) { tie_margin = margin < 0.0f ? 0.0f : margin; }

  void set_sync_mode(Device_Timer::Mode mode) { sync_mode = mode; }
  void set_tests_until_converge(size_t n) { tests_until_converge = n ? n : 1; }
  void set_statistic(Statistic s) { statistic = s; }
  // Extra samples for the variants within `margin` (a fraction) of the fastest; 0 = none.
  void set_refinement(size_t extra_tests, float margin) {
    refine_tests = extra_tests;
    refine_margin = margin < 0.0f ? 0.0f : margin;
  }
  // The reference's exploration: one sample per variant, ranked by the mean, no run-off
  // (reference planning_system.h:53-96).
  void use_reference_defaults() {
    tests_until_converge = 1;
    statistic = MEAN;
    refine_tests = 0;
    tie_margin = 0.0f;
  }
  bool converged(Key key) const { return converged_plans.count(key) != 0; }

  // Run `opts` (or the default variant when the workspace is too small for it).  Until the
  // variant has its samples, an asynchronous timer is upgraded so that earlier work cannot
  // leak into the measurement.  (reference :102-114)
  void execute(Params params, Opts opts, Workspace space, Stream s) {
    const Key key(params);
    const size_t need = executor.calculate_workspace(params, opts);
    if (space.size<char>() < need) opts = degrade_plan(params, opts, space);
    else if (!converged(key)) workspace_seen[key][opts] = need;
    auto sync = sync_mode;
    if (sync == Device_Timer::ASYNCHRONOUS) {
      const size_t samples = tests_until_converge + (converged(key) ? 0 : refine_tests);
      if (executor.get_timings(key)[opts].size() < samples) sync = Device_Timer::SEMI_SYNCHRONOUS;
    }
    executor.execute(params, opts, space, s, sync);
  }

  size_t calculate_workspace(Params params, Opts opts) {
    return executor.calculate_workspace(params, opts);
  }

  Planner_Statistics<Key, Opts> make_statistics() {
    std::map<Key, std::map<Opts, std::vector<float>>> times;
    for (auto& [key, per_opt] : executor.get_timings())
      for (auto& [opt, bank] : per_opt) {
        bank.synchronize();
        times[key][opt] = bank.get_times();
      }
    return Planner_Statistics<Key, Opts>(times);
  }

  // ---- plan persistence (the reference keeps plans in memory only, :55) ---------------------
  // [{"key": <key>, "plan": <variant>}, ...] for every committed plan.
  Json plans_json() {
    Json out = Json::array();
    for (auto& [key, opts] : converged_plans) {
      Json e;
      e["key"] = to_json(key);
      e["plan"] = to_json(opts);
      out.push_back(e);
    }
    return out;
  }
  // Commit plans from plans_json() output, or from a statistics report (json() of
  // make_statistics(): the fastest variant of each key by the current statistic).  Returns
  // the number of plans committed.
  size_t load_plans(const Json& doc) {
    size_t loaded = 0;
    for (const Json& e : doc) {
      Key key = from_json<Key>(e["key"]);
      if (e.contains("plan")) {
        converged_plans.insert_or_assign(key, from_json<Opts>(e["plan"]));
        ++loaded;
      } else if (e.contains("options")) {
        bool any = false;
        Opts best = Opts::default_opts();
        float best_time = std::numeric_limits<float>::max();
        for (const Json& o : e["options"]) {
          Timer_Bank bank;
          for (float ms : o["times"].template get<std::vector<float>>())
            bank.append(Device_Timer(ms));
          if (bank.size() == 0) continue;
          const float t = figure_of(bank);
          if (t < best_time) {
            best = from_json<Opts>(o["option"]);
            best_time = t;
            any = true;
          }
        }
        if (any) {
          converged_plans.insert_or_assign(key, best);
          ++loaded;
        }
      }
    }
    return loaded;
  }
};

using GEMM_Planner = Planning_System<GEMM_Executor<double>>;
using SGEMM_Planner = Planning_System<GEMM_Executor<float>>;

}  // namespace rtat
