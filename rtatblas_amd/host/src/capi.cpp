// extern "C" doors onto the planner classes (include/rtat_planner.h).
#include <cstring>
#include <sstream>
#include <string>
#include <variant>

#include "learned_filter.h"
#include "pattern_filter.h"
#include "planning_system.h"
#include "rtat_planner.h"
#include "syrk.h"
#include "trsm.h"

using namespace rtat;

namespace {

thread_local std::string g_error;

using GemmP = Planning_System<GEMM_Executor<double>>;
using GemmPadP = Planning_System<GEMM_Executor_Pad<double>>;
using GemmTileP = Planning_System<GEMM_Executor_Tile<double>>;
using GemmFusedP = Planning_System<GEMM_Executor_Fused<double>>;
using SyrkP = Planning_System<SYRK_Executor<double>>;
using SyrkFusedP = Planning_System<SYRK_Executor_Fused<double>>;
using TrsmP = Planning_System<TRSM_Executor<double>>;
using TrsmFusedP = Planning_System<TRSM_Executor_Fused<double>>;
using GemmPadTileP = Planning_System<GEMM_Executor_Pad_Tile<double>>;
using SyrkTileP = Planning_System<SYRK_Executor_Tile<double>>;
using TrsmTileP = Planning_System<TRSM_Executor_Tile<double>>;

template <class Opts>
Opts parse_variant(const char* text) {
  std::istringstream in(text);
  Opts o;
  in >> o;
  if (in.fail()) throw std::runtime_error(std::string("malformed variant string: ") + text);
  return o;
}

void copy_out(const std::string& s, char* out, size_t len) {
  if (out == nullptr || len == 0) return;
  std::strncpy(out, s.c_str(), len - 1);
  out[len - 1] = '\0';
}

// Device matrix view over memory the caller owns: the Workspace is sized to the footprint.
Matrix<double> view(const double* p, size_t m, size_t n, size_t ld) {
  return Matrix<double>(Workspace(const_cast<double*>(p), ld * n), m, n, ld);
}

template <class F>
int guarded(F&& f) {
  try {
    return f();
  } catch (const std::exception& e) {
    g_error = e.what();
    return -1;
  } catch (...) {
    g_error = "unknown exception";
    return -1;
  }
}

}  // namespace

struct rtat_planner {
  std::variant<GemmP, GemmPadP, GemmTileP, GemmFusedP, SyrkP, SyrkFusedP, TrsmP, TrsmFusedP,
               GemmPadTileP, SyrkTileP, TrsmTileP>
      impl;
  std::string text;  // storage behind the last *_json() result
  template <class P>
  explicit rtat_planner(std::in_place_type_t<P> t) : impl(t) {}
};

namespace {

GEMM_Inputs<double> gemm_inputs(rtat_handle_t h, int ta, int tb, int m, int n, int k, double alpha,
                                const double* A, int lda, const double* B, int ldb, double beta,
                                double* C, int ldc) {
  const bool at = ta == RTAT_OP_T, bt = tb == RTAT_OP_T;
  return GEMM_Inputs<double>(h, BLAS_Operation((rtat_operation_t)ta),
                             BLAS_Operation((rtat_operation_t)tb),
                             view(A, at ? k : m, at ? m : k, lda),
                             view(B, bt ? n : k, bt ? k : n, ldb), view(C, m, n, ldc), alpha, beta);
}
SYRK_Inputs<double> syrk_inputs(rtat_handle_t h, int uplo, int trans, int n, int k, double alpha,
                                const double* A, int lda, double beta, double* C, int ldc) {
  const bool t = trans == RTAT_OP_T;
  return SYRK_Inputs<double>(h, BLAS_Fill_Mode((rtat_fill_t)uplo),
                             BLAS_Operation((rtat_operation_t)trans),
                             view(A, t ? k : n, t ? n : k, lda), view(C, n, n, ldc), alpha, beta);
}
TRSM_Inputs<double> trsm_inputs(rtat_handle_t h, int side, int uplo, int trans, int diag, int m,
                                int n, double alpha, const double* A, int lda, double* B,
                                int ldb) {
  const size_t na = side == RTAT_SIDE_LEFT ? m : n;
  return TRSM_Inputs<double>(h, BLAS_Side((rtat_side_t)side), BLAS_Fill_Mode((rtat_fill_t)uplo),
                             BLAS_Operation((rtat_operation_t)trans), BLAS_Diag((rtat_diag_t)diag),
                             view(A, na, na, lda), view(B, m, n, ldb), alpha);
}

// create_plan (or the fixed variant), then execute on the handle's stream.
template <class P, class Inputs>
int run_planned(P& planner, Inputs in, const char* variant, void* ws, size_t ws_bytes, char* chosen,
                size_t chosen_len) {
  using Opts = typename P::Opts;
  using Key = typename P::Key;
  Opts opts = variant ? parse_variant<Opts>(variant) : planner.create_plan(Key(in));
  Workspace space((char*)ws, ws_bytes);
  if (space.size<char>() < planner.calculate_workspace(in, opts)) opts = Opts::default_opts();
  gpu::Stream_t raw = nullptr;
  blas_check(gpu::blasGetStream(in.handle, &raw), "blasGetStream");
  planner.execute(in, opts, space, Stream(raw));
  copy_out(std::string(opts), chosen, chosen_len);
  return 0;
}

}  // namespace

namespace {
// The names of the variants the planner's filter admits for `key`, one per line.
template <class KeyT>
const char* admitted_text(rtat_planner_t p, const KeyT& key) {
  if (p == nullptr) return nullptr;
  const int rc = guarded([&] {
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Key, KeyT>) {
        p->text.clear();
        for (auto& o : pl.admitted(key)) p->text += std::string(o) + "\n";
      } else {
        throw std::runtime_error("the planner's method has another kind of problem key");
      }
    }, p->impl);
    return 0;
  });
  return rc == 0 ? p->text.c_str() : nullptr;
}
}  // namespace

extern "C" {

rtat_planner_t rtat_planner_create(const char* method) {
  if (method == nullptr) return nullptr;
  const std::string m(method);
  try {
    if (m == "gemm") return new rtat_planner(std::in_place_type<GemmP>);
    if (m == "gemm_pad") return new rtat_planner(std::in_place_type<GemmPadP>);
    if (m == "gemm_tile") return new rtat_planner(std::in_place_type<GemmTileP>);
    if (m == "gemm_fused") return new rtat_planner(std::in_place_type<GemmFusedP>);
    if (m == "syrk") return new rtat_planner(std::in_place_type<SyrkP>);
    if (m == "syrk_fused") return new rtat_planner(std::in_place_type<SyrkFusedP>);
    if (m == "trsm") return new rtat_planner(std::in_place_type<TrsmP>);
    if (m == "trsm_fused") return new rtat_planner(std::in_place_type<TrsmFusedP>);
    if (m == "gemm_pad_tile") return new rtat_planner(std::in_place_type<GemmPadTileP>);
    if (m == "syrk_tile") return new rtat_planner(std::in_place_type<SyrkTileP>);
    if (m == "trsm_tile") return new rtat_planner(std::in_place_type<TrsmTileP>);
  } catch (const std::exception& e) {
    g_error = e.what();
    return nullptr;
  }
  g_error = "unknown method: " + m;
  return nullptr;
}

void rtat_planner_destroy(rtat_planner_t p) { delete p; }

int rtat_planner_configure(rtat_planner_t p, int tests, int statistic) {
  if (p == nullptr || tests < 1 || statistic < 0 || statistic > 2) return -1;
  std::visit([&](auto& pl) {
    using P = std::decay_t<decltype(pl)>;
    pl.set_tests_until_converge((size_t)tests);
    pl.set_statistic((typename P::Statistic)statistic);
  }, p->impl);
  return 0;
}

int rtat_planner_set_refinement(rtat_planner_t p, int extra_tests, double margin) {
  if (p == nullptr || extra_tests < 0 || !(margin >= 0.0)) return -1;
  std::visit([&](auto& pl) { pl.set_refinement((size_t)extra_tests, (float)margin); }, p->impl);
  return 0;
}

int rtat_planner_set_tie_margin(rtat_planner_t p, double margin) {
  if (p == nullptr || !(margin >= 0.0)) return -1;
  std::visit([&](auto& pl) { pl.set_tie_margin((float)margin); }, p->impl);
  return 0;
}

int rtat_planner_set_filter(rtat_planner_t p, const char* patterns) {
  if (p == nullptr) return -1;
  return guarded([&] {
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if (patterns == nullptr || *patterns == '\0')
        pl.set_filter(Option_Filter<typename P::Key, typename P::Opts>());
      else
        pl.set_filter(pattern_filter<typename P::Key, typename P::Opts>(patterns));
    }, p->impl);
    return 0;
  });
}

int rtat_planner_learn_filter(rtat_planner_t p, const char* stats_json, double slack) {
  if (p == nullptr || stats_json == nullptr || !(slack >= 0.0)) return -1;
  return guarded([&] {
    const Json doc = Json::parse(std::string(stats_json));
    return std::visit([&](auto& pl) -> int {
      using P = std::decay_t<decltype(pl)>;
      using Key = typename P::Key;
      using Opts = typename P::Opts;
      std::map<Key, std::map<Opts, std::vector<float>>> times;
      for (const Json& e : doc) {
        const Key key = from_json<Key>(e["key"]);
        for (const Json& o : e["options"])
          times[key][from_json<Opts>(o["option"])] = o["times"].template get<std::vector<float>>();
      }
      Planner_Statistics<Key, Opts> stats(times);
      pl.set_filter(learn_filter<Key, Opts>(stats, (float)slack));
      return (int)times.size();
    }, p->impl);
  });
}

int rtat_planner_use_reference_defaults(rtat_planner_t p) {
  if (p == nullptr) return -1;
  std::visit([](auto& pl) { pl.use_reference_defaults(); }, p->impl);
  return 0;
}

int rtat_planner_variant_count(rtat_planner_t p) {
  if (p == nullptr) return -1;
  return std::visit([](auto& pl) {
    using P = std::decay_t<decltype(pl)>;
    return (int)P::Opts::enumerate().size();
  }, p->impl);
}

int rtat_planner_variant_name(rtat_planner_t p, int i, char* out, size_t out_len) {
  if (p == nullptr) return -1;
  return std::visit([&](auto& pl) {
    using P = std::decay_t<decltype(pl)>;
    auto all = P::Opts::enumerate();
    if (i < 0 || i >= (int)all.size()) return -1;
    copy_out(std::string(all[i]), out, out_len);
    return 0;
  }, p->impl);
}

const char* rtat_planner_gemm_admitted(rtat_planner_t p, int ta, int tb, int m, int n, int k) {
  return admitted_text(p, GEMM_Key(BLAS_Operation((rtat_operation_t)ta),
                                   BLAS_Operation((rtat_operation_t)tb), m, k, n));
}
const char* rtat_planner_syrk_admitted(rtat_planner_t p, int uplo, int trans, int n, int k) {
  return admitted_text(p, SYRK_Key(BLAS_Fill_Mode((rtat_fill_t)uplo),
                                   BLAS_Operation((rtat_operation_t)trans), n, k));
}
const char* rtat_planner_trsm_admitted(rtat_planner_t p, int side, int uplo, int trans, int diag,
                                       int m, int n) {
  return admitted_text(p, TRSM_Key(BLAS_Side((rtat_side_t)side), BLAS_Fill_Mode((rtat_fill_t)uplo),
                                   BLAS_Operation((rtat_operation_t)trans),
                                   BLAS_Diag((rtat_diag_t)diag), m, n));
}

long long rtat_planner_gemm_workspace(rtat_planner_t p, const char* variant, int ta, int tb, int m,
                                      int n, int k, int lda, int ldb, int ldc) {
  if (p == nullptr || variant == nullptr) return -1;
  long long bytes = -1;
  guarded([&] {
    auto in = gemm_inputs(nullptr, ta, tb, m, n, k, 1.0, nullptr, lda, nullptr, ldb, 0.0, nullptr, ldc);
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, GEMM_Inputs<double>>)
        bytes = (long long)pl.calculate_workspace(in, parse_variant<typename P::Opts>(variant));
      else
        throw std::runtime_error("not a gemm planner");
    }, p->impl);
    return 0;
  });
  return bytes;
}

long long rtat_planner_gemm_workspace_max(rtat_planner_t p, int ta, int tb, int m, int n, int k,
                                          int lda, int ldb, int ldc) {
  if (p == nullptr) return -1;
  long long bytes = -1;
  guarded([&] {
    auto in = gemm_inputs(nullptr, ta, tb, m, n, k, 1.0, nullptr, lda, nullptr, ldb, 0.0, nullptr, ldc);
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, GEMM_Inputs<double>>) {
        size_t most = 0;
        for (auto& o : P::Opts::enumerate()) most = std::max(most, pl.calculate_workspace(in, o));
        bytes = (long long)most;
      } else {
        throw std::runtime_error("not a gemm planner");
      }
    }, p->impl);
    return 0;
  });
  return bytes;
}

long long rtat_planner_syrk_workspace(rtat_planner_t p, const char* variant, int uplo, int trans,
                                      int n, int k, int lda, int ldc) {
  if (p == nullptr || variant == nullptr) return -1;
  long long bytes = -1;
  guarded([&] {
    auto in = syrk_inputs(nullptr, uplo, trans, n, k, 1.0, nullptr, lda, 0.0, nullptr, ldc);
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, SYRK_Inputs<double>>)
        bytes = (long long)pl.calculate_workspace(in, parse_variant<typename P::Opts>(variant));
      else
        throw std::runtime_error("not a syrk planner");
    }, p->impl);
    return 0;
  });
  return bytes;
}

long long rtat_planner_trsm_workspace(rtat_planner_t p, const char* variant, int side, int uplo,
                                      int trans, int diag, int m, int n, int lda, int ldb) {
  if (p == nullptr || variant == nullptr) return -1;
  long long bytes = -1;
  guarded([&] {
    auto in = trsm_inputs(nullptr, side, uplo, trans, diag, m, n, 1.0, nullptr, lda, nullptr, ldb);
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, TRSM_Inputs<double>>)
        bytes = (long long)pl.calculate_workspace(in, parse_variant<typename P::Opts>(variant));
      else
        throw std::runtime_error("not a trsm planner");
    }, p->impl);
    return 0;
  });
  return bytes;
}

long long rtat_planner_syrk_workspace_max(rtat_planner_t p, int uplo, int trans, int n, int k,
                                          int lda, int ldc) {
  if (p == nullptr) return -1;
  long long bytes = -1;
  guarded([&] {
    auto in = syrk_inputs(nullptr, uplo, trans, n, k, 1.0, nullptr, lda, 0.0, nullptr, ldc);
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, SYRK_Inputs<double>>) {
        size_t most = 0;
        for (auto& o : P::Opts::enumerate()) most = std::max(most, pl.calculate_workspace(in, o));
        bytes = (long long)most;
      } else {
        throw std::runtime_error("not a syrk planner");
      }
    }, p->impl);
    return 0;
  });
  return bytes;
}

long long rtat_planner_trsm_workspace_max(rtat_planner_t p, int side, int uplo, int trans, int diag,
                                          int m, int n, int lda, int ldb) {
  if (p == nullptr) return -1;
  long long bytes = -1;
  guarded([&] {
    auto in = trsm_inputs(nullptr, side, uplo, trans, diag, m, n, 1.0, nullptr, lda, nullptr, ldb);
    std::visit([&](auto& pl) {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, TRSM_Inputs<double>>) {
        size_t most = 0;
        for (auto& o : P::Opts::enumerate()) most = std::max(most, pl.calculate_workspace(in, o));
        bytes = (long long)most;
      } else {
        throw std::runtime_error("not a trsm planner");
      }
    }, p->impl);
    return 0;
  });
  return bytes;
}

int rtat_planner_gemm(rtat_planner_t p, rtat_handle_t h, const char* variant, int ta, int tb, int m,
                      int n, int k, double alpha, const double* A, int lda, const double* B,
                      int ldb, double beta, double* C, int ldc, void* ws, size_t ws_bytes,
                      char* chosen, size_t chosen_len) {
  if (p == nullptr || h == nullptr) return -2;
  return guarded([&] {
    auto in = gemm_inputs(h, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
    return std::visit([&](auto& pl) -> int {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, GEMM_Inputs<double>>)
        return run_planned(pl, in, variant, ws, ws_bytes, chosen, chosen_len);
      else
        throw std::runtime_error("not a gemm planner");
    }, p->impl);
  });
}

int rtat_planner_syrk(rtat_planner_t p, rtat_handle_t h, const char* variant, int uplo, int trans,
                      int n, int k, double alpha, const double* A, int lda, double beta, double* C,
                      int ldc, void* ws, size_t ws_bytes, char* chosen, size_t chosen_len) {
  if (p == nullptr || h == nullptr) return -2;
  return guarded([&] {
    auto in = syrk_inputs(h, uplo, trans, n, k, alpha, A, lda, beta, C, ldc);
    return std::visit([&](auto& pl) -> int {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, SYRK_Inputs<double>>)
        return run_planned(pl, in, variant, ws, ws_bytes, chosen, chosen_len);
      else
        throw std::runtime_error("not a syrk planner");
    }, p->impl);
  });
}

int rtat_planner_trsm(rtat_planner_t p, rtat_handle_t h, const char* variant, int side, int uplo,
                      int trans, int diag, int m, int n, double alpha, const double* A, int lda,
                      double* B, int ldb, void* ws, size_t ws_bytes, char* chosen,
                      size_t chosen_len) {
  if (p == nullptr || h == nullptr) return -2;
  return guarded([&] {
    auto in = trsm_inputs(h, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb);
    return std::visit([&](auto& pl) -> int {
      using P = std::decay_t<decltype(pl)>;
      if constexpr (std::is_same_v<typename P::Params, TRSM_Inputs<double>>)
        return run_planned(pl, in, variant, ws, ws_bytes, chosen, chosen_len);
      else
        throw std::runtime_error("not a trsm planner");
    }, p->impl);
  });
}

const char* rtat_planner_stats_json(rtat_planner_t p) {
  if (p == nullptr) return nullptr;
  const int rc = guarded([&] {
    p->text = std::visit([](auto& pl) { return pl.make_statistics().json().dump(2); }, p->impl);
    return 0;
  });
  return rc == 0 ? p->text.c_str() : nullptr;
}

const char* rtat_planner_plans_json(rtat_planner_t p) {
  if (p == nullptr) return nullptr;
  const int rc = guarded([&] {
    p->text = std::visit([](auto& pl) { return pl.plans_json().dump(2); }, p->impl);
    return 0;
  });
  return rc == 0 ? p->text.c_str() : nullptr;
}

int rtat_planner_load_plans(rtat_planner_t p, const char* json_text) {
  if (p == nullptr || json_text == nullptr) return -2;
  return guarded([&] {
    Json doc = Json::parse(std::string(json_text));
    return (int)std::visit([&](auto& pl) { return pl.load_plans(doc); }, p->impl);
  });
}

const char* rtat_planner_last_error(void) { return g_error.c_str(); }

}  // extern "C"
