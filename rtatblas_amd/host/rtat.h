// rtat::rtat — one object holding a lazily built planner per routine and precision
// (reference src/rtat.h).
#pragma once
#include <gemm.h>
#include <planning_system.h>
#include <syrk.h>
#include <trsm.h>

#include <memory>
#include <type_traits>

namespace rtat {

// Built on first use.
template <typename T>
class Lazy {
  std::unique_ptr<T> val;

 public:
  operator T&() {
    if (!val) val = std::make_unique<T>();
    return *val;
  }
};

class rtat {
  Lazy<Planning_System<GEMM_Executor<double>>> dgemm_planner;
  Lazy<Planning_System<GEMM_Executor<float>>> sgemm_planner;
  Lazy<Planning_System<TRSM_Executor<double>>> dtrsm_planner;
  Lazy<Planning_System<TRSM_Executor<float>>> strsm_planner;
  Lazy<Planning_System<SYRK_Executor<double>>> dsyrk_planner;
  Lazy<Planning_System<SYRK_Executor<float>>> ssyrk_planner;

  template <typename T>
  static constexpr void only_real() {
    static_assert(std::is_same_v<T, double> || std::is_same_v<T, float>,
                  "rtat planners exist for double and float");
  }

 public:
  // gemm_planner<double>() / gemm_planner<float>(), and likewise for trsm and syrk.
  template <typename T>
  Planning_System<GEMM_Executor<T>>& gemm_planner() {
    only_real<T>();
    if constexpr (std::is_same_v<T, double>) return dgemm_planner;
    else return sgemm_planner;
  }
  template <typename T>
  Planning_System<TRSM_Executor<T>>& trsm_planner() {
    only_real<T>();
    if constexpr (std::is_same_v<T, double>) return dtrsm_planner;
    else return strsm_planner;
  }
  template <typename T>
  Planning_System<SYRK_Executor<T>>& syrk_planner() {
    only_real<T>();
    if constexpr (std::is_same_v<T, double>) return dsyrk_planner;
    else return ssyrk_planner;
  }
};

}  // namespace rtat
