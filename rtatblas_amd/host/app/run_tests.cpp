// run_tests <file.json>: the JSON-driven driver (reference src/app/run_tests.cpp).  Reads the
// input file, dispatches on method x data_type x run_type, prints the input document with
// "problems" replaced by the timing report.
#include <fstream>
#include <iostream>

#include "planning_system.h"
#include "test_harness.h"

using namespace rtat;

template <typename Executor>
static Json run(const Input_File& file) {
  Test_Harness<Planning_System<Executor>> harness(file.problem_json);
  return file.run_type.val == Run_Type::EXHAUSTIVE ? harness.run_exhaustive(file.repetitions)
                                                   : harness.run_autotune(file.repetitions);
}

template <template <typename> typename Executor>
static Json run_typed(const Input_File& file) {
  return file.data_type.val == Data_Type::FLOAT ? run<Executor<float>>(file)
                                                : run<Executor<double>>(file);
}

static Json dispatch(const Input_File& file) {
  switch (file.method.val) {
    case Method::GEMM: return run_typed<GEMM_Executor>(file);
    case Method::GEMM_PAD: return run_typed<GEMM_Executor_Pad>(file);
    case Method::GEMM_TILE: return run_typed<GEMM_Executor_Tile>(file);
    case Method::SYRK: return run_typed<SYRK_Executor>(file);
    case Method::TRSM: return run_typed<TRSM_Executor>(file);
  }
  throw std::runtime_error("unreachable method");
}

int main(int argc, char* argv[]) {
  if (argc != 2) {
    std::cout << "Expected command line args: filename" << std::endl;
    return 1;
  }
  try {
    std::ifstream in(argv[1]);
    if (!in) throw std::runtime_error(std::string("cannot open ") + argv[1]);
    Json doc = Json::parse(in);
    Input_File file(doc);
    doc["problems"] = dispatch(file);
    std::cout << doc.dump(2) << std::endl;
  } catch (const std::exception& e) {
    std::cerr << "run_tests: " << e.what() << std::endl;
    return 2;
  }
  return 0;
}
