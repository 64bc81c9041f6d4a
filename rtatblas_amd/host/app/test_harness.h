// JSON-driven benchmark harness (reference src/app/test_harness.h): reads a problem list,
// runs every variant (exhaustive) or the planner's choice (autotune) the requested number of
// times, returns the statistics report.
//
// Input file: {"keywords": {"run_type": "exhaustive"|"autotune", "method": "gemm"|"gemm_pad"|
// "gemm_tile"|"gemm_pad_tile"|"gemm_fused"|"syrk"|"syrk_tile"|"syrk_fused"|"trsm"|"trsm_tile"|
// "trsm_fused", "data_type": "double"|"float", "repetitions": N, "filter": "<patterns>"
// (optional: which variants are tried, pattern_filter.h)}, "problems": [<key>, ...]}.
// Beyond the reference, a problem may carry "ld_pad" (extra rows added to every
// leading dimension), "alpha", "beta" and "seed"; operands come from the seeded generator
// (iid uniform[-1,1); symmetric C for syrk; well-conditioned triangular A for trsm) instead
// of an unseeded device RNG.
#pragma once
#include <gemm.h>
#include <gpu-api.h>
#include <json_encoding.h>
#include <mini_json.h>
#include <pattern_filter.h>
#include <syrk.h>
#include <trsm.h>

#include <stdexcept>
#include <vector>

namespace rtat {

namespace detail {
// A keyword with a closed vocabulary; `names[val]` is its spelling.
template <class Names>
class Keyword {
 public:
  int val = 0;
  Keyword(const std::string& s) {
    for (int i = 0; i < (int)Names::count; ++i)
      if (s == Names::names[i]) {
        val = i;
        return;
      }
    throw std::runtime_error(std::string("Invalid ") + Names::what + ": " + s);
  }
  operator std::string() const { return Names::names[val]; }
};
struct Run_Type_Names {
  static constexpr const char* what = "run_type";
  static constexpr size_t count = 2;
  static constexpr const char* names[count] = {"exhaustive", "autotune"};
};
struct Method_Names {
  static constexpr const char* what = "method";
  static constexpr size_t count = 11;
  static constexpr const char* names[count] = {
      "gemm",       "gemm_pad",   "trsm",          "syrk",      "gemm_tile", "gemm_fused",
      "syrk_fused", "trsm_fused", "gemm_pad_tile", "syrk_tile", "trsm_tile"};
};
struct Data_Type_Names {
  static constexpr const char* what = "data_type";
  static constexpr size_t count = 2;
  static constexpr const char* names[count] = {"float", "double"};
};
}  // namespace detail

struct Run_Type : detail::Keyword<detail::Run_Type_Names> {
  enum _Run_Type { EXHAUSTIVE, AUTOTUNE };
  using Keyword::Keyword;
};
struct Method : detail::Keyword<detail::Method_Names> {
  enum _Method {
    GEMM, GEMM_PAD, TRSM, SYRK, GEMM_TILE, GEMM_FUSED, SYRK_FUSED, TRSM_FUSED, GEMM_PAD_TILE,
    SYRK_TILE, TRSM_TILE
  };
  using Keyword::Keyword;
};
struct Data_Type : detail::Keyword<detail::Data_Type_Names> {
  enum _Data_Type { FLOAT, DOUBLE };
  using Keyword::Keyword;
};

// Per-problem extras that are not part of the planner key.
struct Problem_Extras {
  int ld_pad = 0;
  double alpha = 1.0, beta = 0.0;
  uint64_t seed = 1;
  Problem_Extras() = default;
  Problem_Extras(const Json& j)
      : ld_pad(j.value<int>("ld_pad", 0)), alpha(j.value<double>("alpha", 1.0)),
        beta(j.value<double>("beta", 0.0)), seed((uint64_t)j.value<long long>("seed", 1)) {}
};

template <typename Key>
class Problem_Set {
  std::vector<Key> problems;
  std::vector<Problem_Extras> extras;

 public:
  Problem_Set(const Json& json) {
    for (const Json& p : json) {
      problems.push_back(from_json<Key>(p));
      extras.emplace_back(p);
    }
  }
  const std::vector<Key>& get_problems() const { return problems; }
  const Problem_Extras& get_extras(size_t i) const { return extras[i]; }
};

struct Input_File {
  const Json problem_json;
  const Run_Type run_type;
  const Method method;
  const Data_Type data_type;
  const int repetitions;
  const std::string filter;  // variant-name patterns; empty: every variant

  Input_File(const Json& in)
      : problem_json(in["problems"]), run_type(in["keywords"]["run_type"].get<std::string>()),
        method(in["keywords"]["method"].get<std::string>()),
        data_type(in["keywords"]["data_type"].get<std::string>()),
        repetitions(in["keywords"]["repetitions"].get<int>()),
        filter(in["keywords"].value<std::string>("filter", "")) {}
};

// Stream, handle bound to it, operand memory and scratch memory for one run.
struct Device_Resources {
  Stream s;
  gpu::blasHandle_t handle = nullptr;
  ManagedWorkspace scratch_space;

  Device_Resources() : scratch_space(1024), space(1024) {
    blas_check(gpu::blasCreate(&handle), "blasCreate");
    blas_check(gpu::blasSetStream(handle, s), "blasSetStream");
  }
  ~Device_Resources() { gpu::blasDestroy(handle); }
  void sync() { s.synchronize(); }

  // One allocation cut into 512-byte aligned pieces, one per matrix (reference :155-184).
  // The matrices are left uninitialised; fill<T>() gives them contents.
  template <typename T>
  std::vector<Matrix<T>> allocate_matrices(const std::vector<MatrixDims>& dims) {
    std::vector<size_t> bytes;
    size_t total = 0;
    for (auto& d : dims) {
      bytes.push_back((d.footprint() * sizeof(T) + 511) / 512 * 512);
      total += bytes.back();
    }
    space.grow_to_fit<char>(total);
    std::vector<Matrix<T>> out;
    size_t offset = 0;
    for (size_t i = 0; i < dims.size(); ++i) {
      out.emplace_back(Workspace(space, offset, bytes[i]), dims[i]);
      offset += bytes[i];
    }
    return out;
  }

  template <typename T>
  void fill(Matrix<T> A, uint64_t seed, int kind) {
    const auto d = A.dims();
    if constexpr (std::is_same_v<T, double>)
      blas_check(rtat_dfill(handle, A.ptr(), (int)d.m, (int)d.n, (int)d.ld, seed, kind), "dfill");
    else
      blas_check(rtat_sfill(handle, A.ptr(), (int)d.m, (int)d.n, (int)d.ld, seed, kind), "sfill");
  }

 private:
  ManagedWorkspace space;
};

template <typename Planner_Type>
class Test_Harness {
  using Params = typename Planner_Type::Params;
  using Key = typename Planner_Type::Key;
  using Opts = typename Planner_Type::Opts;
  using Scalar = typename Params::Scalar;

  Problem_Set<Key> problems;
  std::string filter;
  Device_Resources resources;

  void run_once(Planner_Type& planner, const Key& problem, const Problem_Extras& ex, Opts opts) {
    Params input = form_input<Scalar>(problem, ex);
    resources.scratch_space.grow_to_fit<char>(planner.calculate_workspace(input, opts));
    planner.execute(input, opts, resources.scratch_space, resources.s);
    resources.sync();
  }

  // Untimed runs of the plain variant on freshly generated operands until the device has
  // been busy for WARM_MS: the clocks of an idle GPU take tens of milliseconds of work to
  // come up, which would otherwise be charged to whichever variant a problem times first
  // (measured here: the first three 8 ms runs of a problem 24 %, 12 % and 7 % slow).  No
  // counterpart in the reference, whose reports carry that bias.
  static constexpr float WARM_MS = 100.0f;
  void warm_up(const Key& problem, const Problem_Extras& ex) {
    float busy_ms = 0.0f;
    for (int i = 0; i < 50 && busy_ms < WARM_MS; ++i) {
      Params input = form_input<Scalar>(problem, ex);
      Device_Timer timer(
          [&](const Stream&) {
            Opts::default_opts().form_operation(input)->execute(resources.handle, Workspace(),
                                                                Workspace());
          },
          resources.s, Device_Timer::SYNCHRONOUS);
      busy_ms += timer.time();
    }
  }

 public:
  Test_Harness(const Json& problem_json, const std::string& filter = "")
      : problems(problem_json), filter(filter) {}

  // problem x variant x repetition; operands are regenerated before every run, outside the
  // timed region (reference :199-214).
  Json run_exhaustive(int repetitions) {
    Planner_Type planner;
    if (!filter.empty()) planner.set_filter(pattern_filter<Key, Opts>(filter));
    for (size_t p = 0; p < problems.get_problems().size(); ++p) {
      warm_up(problems.get_problems()[p], problems.get_extras(p));
      for (auto& opts : planner.admitted(problems.get_problems()[p]))
        for (int i = 0; i < repetitions; ++i)
          run_once(planner, problems.get_problems()[p], problems.get_extras(p), opts);
    }
    return planner.make_statistics().json();
  }

  // problem x repetition, each run using the planner's current choice (reference :216-231).
  Json run_autotune(int repetitions) {
    Planner_Type planner;
    if (!filter.empty()) planner.set_filter(pattern_filter<Key, Opts>(filter));
    for (size_t p = 0; p < problems.get_problems().size(); ++p) {
      const Key& problem = problems.get_problems()[p];
      warm_up(problem, problems.get_extras(p));
      for (int i = 0; i < repetitions; ++i)
        run_once(planner, problem, problems.get_extras(p), planner.create_plan(problem));
    }
    return planner.make_statistics().json();
  }

  // Operand shapes per key (reference :233-277): every matrix as tall as its row count plus
  // the problem's ld_pad.
  template <typename T>
  GEMM_Inputs<T> form_input(GEMM_Key key, const Problem_Extras& ex = Problem_Extras()) {
    const bool an = key.transa == gpu::BLAS_OP_N, bn = key.transb == gpu::BLAS_OP_N;
    const size_t ar = an ? key.m : key.k, ac = an ? key.k : key.m;
    const size_t br = bn ? key.k : key.n, bc = bn ? key.n : key.k;
    auto mats = resources.allocate_matrices<T>({MatrixDims(ar, ac, ar + ex.ld_pad),
                                                MatrixDims(br, bc, br + ex.ld_pad),
                                                MatrixDims(key.m, key.n, key.m + ex.ld_pad)});
    resources.fill(mats[0], ex.seed, RTAT_FILL_IID);
    resources.fill(mats[1], ex.seed + 1, RTAT_FILL_IID);
    resources.fill(mats[2], ex.seed + 2, RTAT_FILL_IID);
    return GEMM_Inputs<T>(resources.handle, key.transa, key.transb, mats[0], mats[1], mats[2],
                          (T)ex.alpha, (T)ex.beta);
  }

  template <typename T>
  TRSM_Inputs<T> form_input(TRSM_Key key, const Problem_Extras& ex = Problem_Extras()) {
    const size_t na = key.side == gpu::BLAS_SIDE_LEFT ? key.m : key.n;
    auto mats = resources.allocate_matrices<T>(
        {MatrixDims(na, na, na + ex.ld_pad), MatrixDims(key.m, key.n, key.m + ex.ld_pad)});
    // Both triangles well conditioned and finite: the transposing variants copy all of A.
    resources.fill(mats[0], ex.seed, RTAT_FILL_TRI_FULL);
    resources.fill(mats[1], ex.seed + 1, RTAT_FILL_IID);
    return TRSM_Inputs<T>(resources.handle, key.side, key.uplo, key.trans, key.diag, mats[0],
                          mats[1], (T)ex.alpha);
  }

  template <typename T>
  SYRK_Inputs<T> form_input(SYRK_Key key, const Problem_Extras& ex = Problem_Extras()) {
    const bool an = key.trans == gpu::BLAS_OP_N;
    const size_t ar = an ? key.n : key.k, ac = an ? key.k : key.n;
    auto mats = resources.allocate_matrices<T>(
        {MatrixDims(ar, ac, ar + ex.ld_pad), MatrixDims(key.n, key.n, key.n + ex.ld_pad)});
    resources.fill(mats[0], ex.seed, RTAT_FILL_IID);
    resources.fill(mats[1], ex.seed + 2, RTAT_FILL_SYMMETRIC);
    return SYRK_Inputs<T>(resources.handle, key.uplo, key.trans, mats[0], mats[1], (T)ex.alpha,
                          (T)ex.beta);
  }

};

}  // namespace rtat
