// rtat::rtat — the facade: one autotuning planner per routine and precision, each built the
// first time it is asked for (reference src/rtat.h:10-60).
#pragma once
#include <gemm.h>
#include <planning_system.h>
#include <syrk.h>
#include <trsm.h>

#include <memory>
#include <tuple>

namespace rtat {

// A value that is constructed on first use.
template <typename T>
class Lazy {
  std::unique_ptr<T> made;

 public:
  T& get() {
    if (!made) made = std::make_unique<T>();
    return *made;
  }
  operator T&() { return get(); }
  bool built() const { return made != nullptr; }
};

class rtat {
  // One slot per planner type; asking for a planner of any other element type fails to
  // compile at the std::get below.
  template <typename... Executors>
  using Slots = std::tuple<Lazy<Planning_System<Executors>>...>;
  Slots<GEMM_Executor<double>, GEMM_Executor<float>, SYRK_Executor<double>, SYRK_Executor<float>,
        TRSM_Executor<double>, TRSM_Executor<float>>
      planners;

  template <typename Executor>
  Planning_System<Executor>& planner_of() {
    return std::get<Lazy<Planning_System<Executor>>>(planners).get();
  }

 public:
  // gemm_planner<double>() / gemm_planner<float>(), and likewise for syrk and trsm.
  template <typename T>
  Planning_System<GEMM_Executor<T>>& gemm_planner() {
    return planner_of<GEMM_Executor<T>>();
  }
  template <typename T>
  Planning_System<SYRK_Executor<T>>& syrk_planner() {
    return planner_of<SYRK_Executor<T>>();
  }
  template <typename T>
  Planning_System<TRSM_Executor<T>>& trsm_planner() {
    return planner_of<TRSM_Executor<T>>();
  }
};

}  // namespace rtat
