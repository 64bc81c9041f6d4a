// run_tests <file.json>: the JSON-driven benchmark driver (reference src/app/run_tests.cpp).
// Reads the input file, picks the harness for its method and element type from a table, and
// prints the input document with "problems" replaced by the timing report.
#include <fstream>
#include <iostream>

#include "planning_system.h"
#include "test_harness.h"

using namespace rtat;

namespace {

using Runner = Json (*)(const Input_File&);

template <typename Executor>
Json run(const Input_File& file) {
  Test_Harness<Planning_System<Executor>> harness(file.problem_json, file.filter);
  if (file.run_type.val == Run_Type::EXHAUSTIVE) return harness.run_exhaustive(file.repetitions);
  return harness.run_autotune(file.repetitions);
}

// One row per method: its runner for each element type, indexed by Data_Type's value.
struct Method_Row {
  int method;
  Runner by_type[2];
};
template <template <typename> typename Executor>
constexpr Method_Row row(int method) {
  Method_Row r{method, {}};
  r.by_type[Data_Type::FLOAT] = &run<Executor<float>>;
  r.by_type[Data_Type::DOUBLE] = &run<Executor<double>>;
  return r;
}
const Method_Row methods[] = {
    row<GEMM_Executor>(Method::GEMM),           row<GEMM_Executor_Pad>(Method::GEMM_PAD),
    row<GEMM_Executor_Tile>(Method::GEMM_TILE), row<SYRK_Executor>(Method::SYRK),
    row<TRSM_Executor>(Method::TRSM),           row<GEMM_Executor_Fused>(Method::GEMM_FUSED),
    row<SYRK_Executor_Fused>(Method::SYRK_FUSED), row<TRSM_Executor_Fused>(Method::TRSM_FUSED),
    row<GEMM_Executor_Pad_Tile>(Method::GEMM_PAD_TILE), row<SYRK_Executor_Tile>(Method::SYRK_TILE),
    row<TRSM_Executor_Tile>(Method::TRSM_TILE),
};

Json report_for(const Input_File& file) {
  for (const Method_Row& r : methods)
    if (r.method == file.method.val) return r.by_type[file.data_type.val](file);
  throw std::runtime_error("no harness for method " + std::string(file.method));
}

}  // namespace

int main(int argc, char* argv[]) {
  if (argc != 2) {
    std::cout << "Expected command line args: filename" << std::endl;
    return 1;
  }
  try {
    std::ifstream in(argv[1]);
    if (!in) throw std::runtime_error(std::string("cannot open ") + argv[1]);
    Json doc = Json::parse(in);
    doc["problems"] = report_for(Input_File(doc));
    std::cout << doc.dump(2) << std::endl;
  } catch (const std::exception& e) {
    std::cerr << "run_tests: " << e.what() << std::endl;
    return 2;
  }
  return 0;
}
