// C++ tests of the host layer (gpu-api, timing, workspace, matrix-op tree, methods, planner,
// JSON codecs), modelled one-for-one on the reference's GoogleTest suites:
//   tests/api_test.cpp, timing_test.cpp, workspace_test.cpp, matrixop_test.cpp,
//   executor_test.cpp, planning_test.cpp, json_test.cpp.
// Host checks use the CPU oracle (oracle/rtat_oracle.h), as the reference's use the loops in
// tests/common.h.  Tests that need no device run with `--cpu`; the rest with `--gpu`.
#include <chrono>
#include <cstring>
#include <random>
#include <set>
#include <sstream>
#include <thread>

#include "json_encoding.h"
#include "learned_filter.h"
#include "mini_test.h"
#include "pattern_filter.h"
#include "planning_system.h"
#include "rtat.h"
#include "rtat_oracle.h"
#include "rtat_planner.h"
#include "test_harness.h"

using namespace rtat;

// ---------------------------------------------------------------------------------------------
// fixtures
// ---------------------------------------------------------------------------------------------
struct Blas_Fixture {
  Stream s;
  gpu::blasHandle_t handle = nullptr;
  Blas_Fixture() {
    blas_check(gpu::blasCreate(&handle), "blasCreate");
    blas_check(gpu::blasSetStream(handle, s), "blasSetStream");
  }
  ~Blas_Fixture() { gpu::blasDestroy(handle); }
};

// Host vector + device copy of an m x n matrix with leading dimension ld
// (the role of TestMatrix in the reference's tests/common.h:24-156).
template <typename T>
struct TestMatrix {
  size_t m, n, ld;
  ManagedWorkspace space;
  std::vector<T> host;

  TestMatrix(size_t m, size_t n) : TestMatrix(m, n, m) {}
  TestMatrix(size_t m, size_t n, size_t ld)
      : m(m), n(n), ld(ld), space(std::max<size_t>(ld * n, 1) * sizeof(T)), host(ld * n) {
    static std::mt19937_64 engine(20240607);
    std::uniform_real_distribution<T> unif(-1.0, 1.0);
    for (auto& x : host) x = unif(engine);
    upload();
  }
  void upload() {
    if (!host.empty())
      gpuAssert(gpu::Memcpy(space, host.data(), host.size() * sizeof(T), gpu::MemcpyHostToDevice));
  }
  void download() {
    if (!host.empty())
      gpuAssert(gpu::Memcpy(host.data(), space, host.size() * sizeof(T), gpu::MemcpyDeviceToHost));
  }
  T& at(size_t i, size_t j) { return host[j * ld + i]; }
  Matrix<T> matrix() { return Matrix<T>(space, m, n, ld); }
  operator Matrix<T>() { return matrix(); }
  Workspace workspace() { return space; }
  T max_abs() {
    T v = 0;
    for (size_t j = 0; j < n; ++j)
      for (size_t i = 0; i < m; ++i) v = std::max(v, std::abs(at(i, j)));
    return v;
  }
  bool is_zero(T eps = std::is_same_v<T, float> ? T(1e-4) : T(1e-10)) { return max_abs() <= eps; }
};

template <typename T>
static T max_diff(TestMatrix<T>& A, TestMatrix<T>& B) {
  T d = 0;
  for (size_t j = 0; j < A.n; ++j)
    for (size_t i = 0; i < A.m; ++i) d = std::max(d, std::abs(A.at(i, j) - B.at(i, j)));
  return d;
}

// Host GEMM / TRSM on TestMatrix: the oracle in double, a plain loop in float.
template <typename T>
static void host_gemm(TestMatrix<T>& A, TestMatrix<T>& B, TestMatrix<T>& C, T alpha, T beta,
                      bool ta, bool tb) {
  const int k = (int)(ta ? A.m : A.n);
  if constexpr (std::is_same_v<T, double>) {
    orc_dgemm(ta ? ORC_OP_T : ORC_OP_N, tb ? ORC_OP_T : ORC_OP_N, (int)C.m, (int)C.n, k, alpha,
              A.host.data(), (int)A.ld, B.host.data(), (int)B.ld, beta, C.host.data(), (int)C.ld);
  } else {
    for (size_t j = 0; j < C.n; ++j)
      for (size_t i = 0; i < C.m; ++i) {
        double acc = 0;
        for (int l = 0; l < k; ++l)
          acc += (double)(ta ? A.at(l, i) : A.at(i, l)) * (double)(tb ? B.at(j, l) : B.at(l, j));
        C.at(i, j) = (T)(alpha * acc + (beta == 0 ? 0.0 : beta * C.at(i, j)));
      }
  }
}

static void make_triangular(TestMatrix<double>& A, bool lower, bool unit, double boost,
                            double shrink) {
  for (size_t j = 0; j < A.n; ++j)
    for (size_t i = 0; i < A.m; ++i) {
      if ((lower && i < j) || (!lower && i > j)) A.at(i, j) = 0.0;
      else if (i == j) A.at(i, j) = unit ? 1.0 : A.at(i, j) + boost;
      else A.at(i, j) /= shrink;
    }
}

// ---------------------------------------------------------------------------------------------
// api_test.cpp
// ---------------------------------------------------------------------------------------------
TEST(API, Creation, true) {
  Stream s;
  Event e;
  Stream copy = s;
  CHECK((gpu::Stream_t)copy == (gpu::Stream_t)s);
}

TEST(API, Elapsed_Time, true) {
  Event e1, e2;
  Stream st;
  double *x, *y;
  gpuAssert(gpu::Malloc(&x, 512));
  gpuAssert(gpu::Malloc(&y, 512));
  e1.record(st);
  gpuAssert(gpu::MemcpyAsync(y, x, 512, gpu::MemcpyDeviceToDevice, st));
  e2.record(st);
  gpuAssert(gpu::DeviceSynchronize());
  const float ms = Event::elapsed_time(e1, e2);
  CHECK(ms >= 0.0f && ms < 1000.0f);
  gpuAssert(gpu::Free(x));
  gpuAssert(gpu::Free(y));
}

TEST(API, String_Rep, false) {
  CHECK_EQ(std::string(BLAS_Operation(gpu::BLAS_OP_T)), std::string("T"));
  CHECK(BLAS_Operation("N") == gpu::BLAS_OP_N);
  CHECK(!BLAS_Operation("N") == gpu::BLAS_OP_T);
  CHECK_EQ(std::string(BLAS_Fill_Mode("Lower")), std::string("Lower"));
  CHECK(!BLAS_Fill_Mode("Lower") == gpu::BLAS_FILL_MODE_UPPER);
  CHECK(BLAS_Side("Right") == gpu::BLAS_SIDE_RIGHT);
  CHECK_EQ(std::string(BLAS_Diag(gpu::BLAS_DIAG_NON_UNIT)), std::string("Non-Unit"));
  CHECK_THROWS(BLAS_Operation("X"));
  CHECK_THROWS(BLAS_Diag("NonUnit"));
}

TEST(API, Device_RNG_Range, true) {
  Stream s;
  Device_RNG rng(s);
  const size_t len = 5000;
  ManagedWorkspace mem(len * sizeof(double));
  rng.uniform<double>((double*)mem, len);
  s.synchronize();
  std::vector<double> h(len);
  gpuAssert(gpu::Memcpy(h.data(), (double*)mem, len * sizeof(double), gpu::MemcpyDeviceToHost));
  double mean = 0;
  bool in_range = true;
  for (double v : h) {
    in_range = in_range && v > 0.0 && v <= 1.0;
    mean += v / len;
  }
  CHECK(in_range);
  CHECK_NEAR(mean, 0.5, 0.05);
}

// ---------------------------------------------------------------------------------------------
// timing_test.cpp
// ---------------------------------------------------------------------------------------------
TEST(Device_Timer, Time, true) {
  const int interval = 50;
  Stream s;
  for (int i = 0; i < 3; ++i) {
    Device_Timer timer(
        [&](Stream) { std::this_thread::sleep_for(std::chrono::milliseconds(interval)); }, s);
    CHECK_NEAR(timer.time(), interval, 1.5);
  }
}

TEST(Timer_Bank, Times, true) {
  const int interval = 76;
  Timer_Bank timers;
  Stream s;
  for (int i = 0; i < 3; ++i) {
    Device_Timer timer(
        [&](Stream) { std::this_thread::sleep_for(std::chrono::milliseconds(interval)); }, s);
    timers.append(timer);
  }
  CHECK_EQ(timers.size(), (size_t)3);
  s.synchronize();
  CHECK_EQ(timers.completed(), (size_t)3);
  for (float t : timers.get_times()) CHECK_NEAR(t, interval, 1.5);
}

TEST(Timer_Bank, Known_Times_And_Statistics, false) {
  Timer_Bank bank;
  for (float t : {5.f, 1.f, 3.f}) bank.append(Device_Timer(t));
  CHECK_EQ(bank.size(), (size_t)3);
  bank.synchronize();
  CHECK_EQ(bank.completed(), (size_t)3);
  CHECK_NEAR(bank.mean(), 3.0, 1e-6);
  CHECK_NEAR(bank.median(), 3.0, 1e-6);
  CHECK_NEAR(bank.minimum(), 1.0, 1e-6);
}

// ---------------------------------------------------------------------------------------------
// workspace_test.cpp (host memory only)
// ---------------------------------------------------------------------------------------------
TEST(Workspace, Constructors_And_Size, false) {
  Workspace empty;
  CHECK_EQ(empty.size<char>(), (size_t)0);
  const size_t N = 8192;
  std::vector<char> bytes(N);
  Workspace space(bytes.data(), N);
  CHECK_EQ(space.size<char>(), N);
  CHECK_EQ(space.size<double>(), N / sizeof(double));
  CHECK_EQ(space.size<int>(), N / sizeof(int));
  CHECK_EQ(space.size<float>(), N / sizeof(float));
}

TEST(Workspace, Offset_Constructor, false) {
  const size_t N = 1024;
  std::vector<char> bytes(N);
  Workspace space(bytes.data(), N);
  Workspace sub(space, 301, 123);
  CHECK((char*)sub == &bytes[301]);
  CHECK_EQ(sub.size<char>(), (size_t)123);
  // the reference dies here (workspace_test.cpp:48); this build throws
  CHECK_THROWS(Workspace(space, N - 2, 10));
}

TEST(Workspace, Peel, false) {
  const size_t N = 1024;
  std::vector<char> bytes(N);
  Workspace space(bytes.data(), N);
  const size_t s1 = 18, s2 = 27, s3 = 48;
  Workspace p1 = space.peel<double>(s1);
  Workspace p2 = space.peel<float>(s2);
  Workspace p3 = space.peel<char>(s3);
  CHECK_EQ(p1.size<char>(), s1 * sizeof(double));
  CHECK((char*)p1 == &bytes[0]);
  CHECK_EQ(p2.size<char>(), s2 * sizeof(float));
  CHECK((char*)p2 == &bytes[s1 * sizeof(double)]);
  CHECK_EQ(p3.size<char>(), s3);
  CHECK((char*)p3 == &bytes[s1 * sizeof(double) + s2 * sizeof(float)]);
  const size_t used = s1 * sizeof(double) + s2 * sizeof(float) + s3;
  CHECK_EQ(space.size<char>(), N - used);
  CHECK((char*)space == &bytes[used]);
  CHECK_THROWS(space.peel<char>(N));
}

TEST(Matrix, Dims_And_Block, false) {
  CHECK_THROWS(MatrixDims(5, 2, 4));
  CHECK_EQ(MatrixDims(5, 3, 8).footprint(), (size_t)24);
  CHECK_EQ(padded_ld(10, 32), (size_t)32);
  CHECK_EQ(padded_ld(64, 32), (size_t)64);
  CHECK_EQ(padded_ld(7, 1), (size_t)7);
  std::vector<double> mem(8 * 6);
  Matrix<double> A(Workspace(mem.data(), mem.size()), 7, 6, 8);
  Matrix<double> b = A.block(2, 3, 4, 2);
  CHECK(b.ptr() == &mem[2 + 3 * 8]);
  CHECK_EQ(b.dims().ld, (size_t)8);
  CHECK_THROWS(A.block(5, 0, 4, 1));
  CHECK(A.at(2, 3) == &mem[2 + 3 * 8]);
  CHECK_EQ(MatrixDims(7, 6, 8).span(), (size_t)(5 * 8 + 7));
  CHECK_EQ(MatrixDims(7, 0, 8).span(), (size_t)0);
  CHECK(MatrixDims(7, 6, 8).transposed() == MatrixDims(6, 7, 6));
  CHECK(MatrixDims(7, 6, 8).transposed(4) == MatrixDims(6, 7, 8));
  CHECK(MatrixDims(7, 6, 8).repadded(32) == MatrixDims(7, 6, 32));
  CHECK(MatrixDims(7, 6, 8) != MatrixDims(7, 6, 7));
}

// ---------------------------------------------------------------------------------------------
// tree shape and workspace accounting without a device
// ---------------------------------------------------------------------------------------------
static Matrix<double> fake(size_t m, size_t n, size_t ld) {
  return Matrix<double>(Workspace((double*)nullptr, ld * n), m, n, ld);
}

TEST(Tree, Workspace_By_Hand_GEMM, false) {
  const size_t m = 70, n = 45, k = 62;
  GEMM_Inputs<double> in(nullptr, gpu::BLAS_OP_N, gpu::BLAS_OP_N, fake(m, k, m), fake(k, n, k),
                         fake(m, n, m), 1.0, 0.0);
  std::map<std::string, size_t> want = {{"NNN", 0},         {"TNN", k * m},
                                        {"NTN", n * k},     {"TTN", k * m + n * k},
                                        {"NNT", n * m},     {"TNT", k * m + n * m},
                                        {"NTT", n * k + n * m}, {"TTT", k * m + n * k + n * m}};
  for (auto& opts : GEMM_Options::enumerate())
    CHECK_EQ(opts.form_operation(in)->workspace_req_bytes(), 8 * want[std::string(opts)]);
  auto up = [](size_t x) { return (x + 31) / 32 * 32; };
  GEMM_Options_Pad pa(BLAS_Op::NOTRANS, Pad_Op::PAD, BLAS_Op::NOTRANS, Pad_Op::NOPAD,
                      BLAS_Op::NOTRANS, Pad_Op::NOPAD);
  CHECK_EQ(pa.form_operation(in)->workspace_req(), up(m) * k);
  GEMM_Options_Pad all(BLAS_Op::TRANS, Pad_Op::PAD, BLAS_Op::TRANS, Pad_Op::PAD, BLAS_Op::TRANS,
                       Pad_Op::PAD);
  CHECK_EQ(all.form_operation(in)->workspace_req(), up(k) * m + up(n) * k + up(n) * m);
  // the oracle's accounting agrees for every pad variant
  for (auto& o : GEMM_Options_Pad::enumerate())
    CHECK_EQ((long)o.form_operation(in)->workspace_req_bytes(),
             orc_gemm_workspace(std::string(o).c_str(), ORC_OP_N, ORC_OP_N, (int)m, (int)n, (int)k,
                                (int)m, (int)k, (int)m));
}

TEST(Tree, Workspace_By_Hand_SYRK_TRSM, false) {
  const size_t n = 213, k = 74;
  SYRK_Inputs<double> si(nullptr, gpu::BLAS_FILL_MODE_LOWER, gpu::BLAS_OP_N, fake(n, k, n),
                         fake(n, n, n), 1.0, 0.0);
  CHECK_EQ(SYRK_Options(false, false).form_operation(si)->workspace_req(), (size_t)0);
  CHECK_EQ(SYRK_Options(true, false).form_operation(si)->workspace_req(), k * n);
  CHECK_EQ(SYRK_Options(false, true).form_operation(si)->workspace_req(), n * n);
  CHECK_EQ(SYRK_Options(true, true).form_operation(si)->workspace_req(), k * n + n * n);
  const size_t m = 435, nn = 527;
  TRSM_Inputs<double> ti(nullptr, gpu::BLAS_SIDE_LEFT, gpu::BLAS_FILL_MODE_LOWER, gpu::BLAS_OP_N,
                         gpu::BLAS_DIAG_NON_UNIT, fake(m, m, m), fake(m, nn, m), 1.0);
  CHECK_EQ(TRSM_Options(false, false).form_operation(ti)->workspace_req(), (size_t)0);
  CHECK_EQ(TRSM_Options(false, true).form_operation(ti)->workspace_req(), m * m);
  CHECK_EQ(TRSM_Options(true, false).form_operation(ti)->workspace_req(), nn * m);
  CHECK_EQ(TRSM_Options(true, true).form_operation(ti)->workspace_req(), m * m + nn * m);
}

TEST(Tree, Shape_Errors_Throw, false) {
  auto leaf = [](size_t m, size_t n) -> std::unique_ptr<MatrixOp<double>> {
    return std::make_unique<NoOp<double>>(fake(m, n, m));
  };
  CHECK_THROWS(MatrixMult<double>(leaf(4, 5), leaf(6, 3), leaf(4, 3), false, false, 1.0, 0.0));
  CHECK_THROWS(MatrixAccumulate<double>(leaf(4, 5), leaf(4, 5), 1.0, 0.0, true));
  CHECK_THROWS(MatrixTrs<double>(leaf(4, 5), leaf(4, 3), true, true, false, false, 1.0));
  CHECK_THROWS(MatrixSyrk<double>(leaf(4, 5), leaf(5, 5), true, false, 1.0, 0.0));
  MatrixMove<double> mv(leaf(10, 12), 1.0, true, 8);
  CHECK_EQ(mv.dims().m, (size_t)12);
  CHECK_EQ(mv.dims().n, (size_t)10);
  CHECK_EQ(mv.dims().ld, (size_t)16);
  CHECK_EQ(mv.output_space_req(), (size_t)160);
}

TEST(Options, Enumeration_Order_And_Strings, false) {
  std::string all;
  for (auto& o : GEMM_Options::enumerate()) all += std::string(o) + " ";
  CHECK_EQ(all, std::string("NNN NNT NTN NTT TNN TNT TTN TTT "));
  CHECK_EQ(GEMM_Options_Pad::enumerate().size(), (size_t)64);
  CHECK_EQ(std::string(GEMM_Options_Pad::enumerate()[1]), std::string("NNNNNP"));
  all.clear();
  for (auto& o : SYRK_Options::enumerate()) all += std::string(o) + " ";
  CHECK_EQ(all, std::string("FF FT TF TT "));
  all.clear();
  for (auto& o : TRSM_Options::enumerate()) all += std::string(o) + " ";
  CHECK_EQ(all, std::string("FF FT TF TT "));
  CHECK_EQ(std::string(GEMM_Key(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 5, 6, 7)), std::string("T,N,,5,6,7"));
  CHECK_EQ(std::string(SYRK_Key(gpu::BLAS_FILL_MODE_LOWER, gpu::BLAS_OP_N, 8, 9)),
           std::string("Lower,N,8,9"));
  CHECK_EQ(std::string(TRSM_Key(gpu::BLAS_SIDE_LEFT, gpu::BLAS_FILL_MODE_UPPER, gpu::BLAS_OP_T,
                                gpu::BLAS_DIAG_NON_UNIT, 3, 4)),
           std::string("Left,Upper,T,Non-Unit,3,4"));
  // stream codecs round-trip (the reference's SYRK / TRSM readers lose the letters)
  for (auto& o : SYRK_Options::enumerate()) {
    std::istringstream in{std::string(o)};
    SYRK_Options back;
    in >> back;
    CHECK_EQ(std::string(back), std::string(o));
  }
  for (auto& o : GEMM_Options_Tile::enumerate()) {
    std::istringstream in{std::string(o)};
    GEMM_Options_Tile back;
    in >> back;
    CHECK_EQ(std::string(back), std::string(o));
  }
  GEMM_Options bad;
  std::istringstream in("NNNN");
  in >> bad;
  CHECK(in.fail());
  CHECK_THROWS(BLAS_Op("X"));
  CHECK_THROWS(Pad_Op("T"));
  CHECK_THROWS(Bool_Op("N"));
}

TEST(Predicates, Combinators, false) {
  Predicate<int> even = [](int x) { return x % 2 == 0; };
  Predicate<int> big = [](int x) { return x > 10; };
  CHECK(conjunction<int>({even, big})(12));
  CHECK(!conjunction<int>({even, big})(4));
  CHECK(disjunction<int>({even, big})(4));
  CHECK(!disjunction<int>({even, big})(3));
  CHECK(conjunction<int>({})(3));
  CHECK(!disjunction<int>({})(3));
  CHECK(negation<int>(even)(3));
  CHECK(!negation<int>(even)(4));
  Option_Filter<GEMM_Key, GEMM_Options> only_plain(
      [](std::pair<GEMM_Options, GEMM_Key> p) { return std::string(p.first)[2] == 'N'; });
  CHECK_EQ(only_plain.apply(GEMM_Key(gpu::BLAS_OP_N, gpu::BLAS_OP_N, 1, 1, 1)).size(), (size_t)4);
}

// ---------------------------------------------------------------------------------------------
// json_test.cpp
// ---------------------------------------------------------------------------------------------
TEST(JSON, Mini_Json_Basics, false) {
  Json j = Json::parse(R"({"b": [1, 2.5, "x\n", true, null], "a": {"k": -3}})");
  CHECK_EQ(j["a"]["k"].get<int>(), -3);
  CHECK_EQ(j["b"].size(), (size_t)5);
  CHECK_NEAR(j["b"][1].get<double>(), 2.5, 0);
  CHECK_EQ(j["b"][2].get<std::string>(), std::string("x\n"));
  CHECK_EQ(j.dump(), std::string(R"({"a":{"k":-3},"b":[1,2.5,"x\n",true,null]})"));
  CHECK(Json::parse(j.dump(2)) == j);
  CHECK_THROWS(Json::parse("{\"a\": }"));
  CHECK_THROWS(j["missing"].get<int>() + (static_cast<const Json&>(j))["missing"].get<int>());
  Json t(std::vector<float>{0.1f, 2.0f});
  CHECK(Json::parse(t.dump())[0].get<float>() == 0.1f);
}

TEST(JSON, SYRK_Key, false) {
  for (auto uplo : {"Lower", "Upper"})
    for (auto trans : {"N", "T"}) {
      Json kj;
      kj["uplo"] = uplo; kj["trans"] = trans; kj["n"] = 6741; kj["k"] = 2463;
      CHECK(to_json(from_json<SYRK_Key>(kj)) == kj);
      SYRK_Key key{BLAS_Fill_Mode(uplo), BLAS_Operation(trans), 6741, 2463};
      SYRK_Key back = from_json<SYRK_Key>(to_json(key));
      CHECK(!(back < key) && !(key < back));
    }
}

TEST(JSON, SYRK_And_TRSM_Options, false) {
  for (auto a : {"T", "F"})
    for (auto c : {"T", "F"}) {
      Json oj;
      oj["transA"] = a; oj["transC"] = c;
      CHECK(to_json(from_json<SYRK_Options>(oj)) == oj);
      Json tj;
      tj["swap_side"] = a; tj["transA"] = c;
      CHECK(to_json(from_json<TRSM_Options>(tj)) == tj);
    }
  for (bool a : {false, true})
    for (bool c : {false, true}) {
      SYRK_Options o(a, c), back = from_json<SYRK_Options>(to_json(o));
      CHECK(!(back < o) && !(o < back));
      TRSM_Options t(a, c), tback = from_json<TRSM_Options>(to_json(t));
      CHECK(!(tback < t) && !(t < tback));
    }
}

TEST(JSON, TRSM_Key, false) {
  for (auto side : {"Left", "Right"})
    for (auto uplo : {"Lower", "Upper"})
      for (auto trans : {"N", "T"})
        for (auto diag : {"Unit", "Non-Unit"}) {
          Json kj;
          kj["side"] = side; kj["uplo"] = uplo; kj["trans"] = trans; kj["diag"] = diag;
          kj["m"] = 10025; kj["n"] = 4001;
          CHECK(to_json(from_json<TRSM_Key>(kj)) == kj);
          TRSM_Key key{BLAS_Side(side), BLAS_Fill_Mode(uplo), BLAS_Operation(trans),
                       BLAS_Diag(diag), 10025, 4001};
          TRSM_Key back = from_json<TRSM_Key>(to_json(key));
          CHECK(!(back < key) && !(key < back));
        }
}

TEST(JSON, GEMM_Key_And_Options, false) {
  for (auto ta : {"N", "T"})
    for (auto tb : {"N", "T"}) {
      Json kj;
      kj["transA"] = ta; kj["transB"] = tb; kj["m"] = 500; kj["n"] = 200; kj["k"] = 900;
      GEMM_Key key = from_json<GEMM_Key>(kj);
      CHECK_EQ(key.m, 500); CHECK_EQ(key.n, 200); CHECK_EQ(key.k, 900);
      CHECK(to_json(key) == kj);
      GEMM_Key made(BLAS_Operation(ta), BLAS_Operation(tb), 500, 900, 200);  // (m, k, n)
      GEMM_Key back = from_json<GEMM_Key>(to_json(made));
      CHECK(!(back < made) && !(made < back));
    }
  for (auto& o : GEMM_Options::enumerate()) {
    GEMM_Options back = from_json<GEMM_Options>(to_json(o));
    CHECK(!(back < o) && !(o < back));
  }
  for (auto ta : {"N", "T"})
    for (auto tb : {"N", "T"})
      for (auto tc : {"N", "T"})
        for (auto pa : {"N", "P"})
          for (auto pb : {"N", "P"})
            for (auto pc : {"N", "P"}) {
              Json oj;
              oj["transA"] = ta; oj["transB"] = tb; oj["transC"] = tc;
              oj["padA"] = pa; oj["padB"] = pb; oj["padC"] = pc;
              GEMM_Options_Pad o = from_json<GEMM_Options_Pad>(oj);
              CHECK(to_json(o) == oj);
              CHECK_EQ(std::string(o), std::string(ta) + tb + tc + pa + pb + pc);
            }
  for (auto& o : GEMM_Options_Tile::enumerate()) {
    GEMM_Options_Tile back = from_json<GEMM_Options_Tile>(to_json(o));
    CHECK(!(back < o) && !(o < back));
  }
  // "auto" comes first, so the default variant - the plain call - is one of the candidates
  CHECK_EQ(to_json(GEMM_Options_Tile::enumerate()[0])["tile"].get<std::string>(),
           std::string("auto"));
  CHECK_EQ(std::string(GEMM_Options_Tile::enumerate()[0]),
           std::string(GEMM_Options_Tile::default_opts()));
}

TEST(JSON, Kernel_Option_Families, false) {
  // The families that add the kernel's own choices to the reference's switches
  // (src/methods/gemm.cpp:28-39, syrk.cpp:28-35, trsm.cpp:29-36): counts, spelling, the default
  // first, and every variant through text and JSON and back.
  CHECK_EQ(GEMM_Options_Tile::enumerate().size(), (size_t)(8 * 5));
  CHECK_EQ(GEMM_Options_Pad_Tile::enumerate().size(), (size_t)(64 * 5 * 3));
  CHECK_EQ(SYRK_Options_Tile::enumerate().size(), (size_t)(4 * 5 * 3));
  CHECK_EQ(TRSM_Options_Tile::enumerate().size(), (size_t)(4 * 5 * 3 * 3));
  CHECK_EQ(std::string(GEMM_Options_Pad_Tile::default_opts()), std::string("NNNNNN/auto/auto"));
  CHECK_EQ(std::string(SYRK_Options_Tile::default_opts()), std::string("FF/auto/auto"));
  CHECK_EQ(std::string(TRSM_Options_Tile::default_opts()), std::string("FF/auto/auto/auto"));
  CHECK_EQ(std::string(GEMM_Options_Pad_Tile::enumerate().back()),
           std::string("TTTPPP/64x64/split"));
  CHECK_EQ(std::string(TRSM_Options_Tile::enumerate().back()), std::string("TT/64x64/split/1024"));
  auto round_trip = [](auto proto) {
    using O = decltype(proto);
    std::set<std::string> names;
    for (auto& o : O::enumerate()) {
      const std::string name = std::string(o);
      CHECK(names.insert(name).second);  // no two variants share a name
      O via_json = from_json<O>(to_json(o));
      CHECK_EQ(std::string(via_json), name);
      O via_text;
      std::istringstream in(name);
      in >> via_text;
      CHECK(!in.fail());
      CHECK_EQ(std::string(via_text), name);
    }
  };
  round_trip(GEMM_Options_Tile());
  round_trip(GEMM_Options_Pad_Tile());
  round_trip(SYRK_Options_Tile());
  round_trip(TRSM_Options_Tile());
  // field vocabulary of the plan files
  Json j = to_json(TRSM_Options_Tile('T', 'F', "128x64", "split", "1024"));
  CHECK_EQ(j["swap_side"].get<std::string>(), std::string("T"));
  CHECK_EQ(j["transA"].get<std::string>(), std::string("F"));
  CHECK_EQ(j["tile"].get<std::string>(), std::string("128x64"));
  CHECK_EQ(j["tail"].get<std::string>(), std::string("split"));
  CHECK_EQ(j["panel"].get<std::string>(), std::string("1024"));
  j = to_json(GEMM_Options_Pad_Tile('N', 'T', 'N', 'P', 'N', 'P', "256x128", "whole"));
  CHECK_EQ(j["padA"].get<std::string>(), std::string("P"));
  CHECK_EQ(j["transB"].get<std::string>(), std::string("T"));
  CHECK_EQ(j["tail"].get<std::string>(), std::string("whole"));
  // malformed texts are refused, unknown names throw
  SYRK_Options_Tile so;
  CHECK(!SYRK_Options_Tile::spell_into(so, "FF"));
  CHECK(!SYRK_Options_Tile::spell_into(so, "FF/auto"));
  CHECK(!SYRK_Options_Tile::spell_into(so, "F/auto/auto"));
  CHECK(!SYRK_Options_Tile::spell_into(so, "FF/auto/auto/auto"));
  CHECK_THROWS(SYRK_Options_Tile::spell_into(so, "FF/96x96/auto"));
  CHECK_THROWS(Tail_Op("sometimes"));
  CHECK_THROWS(Panel_Op("768"));
  CHECK_THROWS(Panel_Op(3));
  // the kernel-options word the trees hand to the *_ex entry points
  CHECK_EQ(RTAT_KERNEL_OPTIONS(RTAT_GEMM_T128x64, RTAT_TAIL_SPLIT, RTAT_PANEL_1024), 3 + 512 + 8192);
  CHECK_EQ(RTAT_KERNEL_OPTIONS_TILE(0x2203), 3);
  CHECK_EQ(RTAT_KERNEL_OPTIONS_TAIL(0x2203), 2);
  CHECK_EQ(RTAT_KERNEL_OPTIONS_PANEL(0x2203), 2);
  // workspace: the kernel options change no tree, so no variant needs more than its letters do
  const size_t m = 100, n = 80, k = 60;
  Matrix<double> A(Workspace(), m, k, m), B(Workspace(), k, n, k), C(Workspace(), m, n, m);
  GEMM_Inputs<double> in(nullptr, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, B, C, 1.0, 0.5);
  for (auto& o : GEMM_Options_Pad_Tile::enumerate()) {
    GEMM_Options_Pad plain(o.transa, o.pada, o.transb, o.padb, o.transc, o.padc);
    GEMM_Options_Pad_Tile copy = o;
    CHECK_EQ(copy.form_operation(in)->workspace_req(), plain.form_operation(in)->workspace_req());
  }
}

// ---------------------------------------------------------------------------------------------
// planner logic with injected timings (no device): Dummy_* as in planning_test.cpp:8-62
// ---------------------------------------------------------------------------------------------
template <typename T>
struct Dummy_Op : MatrixOp<T> {
  Dummy_Op() : MatrixOp<T>({}) {}
  Matrix<T> execute(gpu::blasHandle_t, Workspace, Workspace) override { return Matrix<T>(); }
  size_t output_space_req() const override { return 0; }
  MatrixDims dims() const override { return MatrixDims(); }
};
struct Dummy_Params {
  gpu::blasHandle_t handle;
  int i;
  Dummy_Params(gpu::blasHandle_t handle, int i) : handle(handle), i(i) {}
};
struct Dummy_Key {
  int i;
  Dummy_Key(Dummy_Params p) : i(p.i) {}
  bool operator<(const Dummy_Key& o) const { return i < o.i; }
};
struct Dummy_Opts {
  int i;
  Dummy_Opts(int i = 0) : i(i) {}
  operator std::string() const { return std::to_string(i); }
  static std::vector<Dummy_Opts> enumerate() { return {Dummy_Opts(1), Dummy_Opts(2), Dummy_Opts(3)}; }
  bool operator<(const Dummy_Opts& o) const { return i < o.i; }
  static Dummy_Opts default_opts() { return Dummy_Opts(); }
  std::unique_ptr<MatrixOp<double>> form_operation(Dummy_Params) {
    return std::make_unique<Dummy_Op<double>>();
  }
};
struct Dummy_Executor : Executor<Dummy_Params, Dummy_Key, Dummy_Opts> {
  void warmup(Dummy_Params, Dummy_Opts, Stream) override {}
};
// Records a made-up time per variant instead of touching the device: variant i "takes"
// cost[i] ms (plus a first-call penalty), so the planner's choice is predictable.
struct Fake_Executor : Executor<Dummy_Params, Dummy_Key, Dummy_Opts> {
  std::map<int, float> cost{{1, 5.f}, {2, 2.f}, {3, 9.f}};
  float first_call_penalty = 0.f;
  int calls = 0;
  void warmup(Dummy_Params, Dummy_Opts, Stream) override {}
  void execute(Dummy_Params params, Dummy_Opts opts, Workspace, Stream,
               Device_Timer::Mode = Device_Timer::ASYNCHRONOUS) override {
    Timer_Bank& bank = timer_log[Dummy_Key(params)][opts];
    const float t = cost[opts.i] + (bank.size() == 0 ? first_call_penalty : 0.f);
    bank.append(Device_Timer(t));
    ++calls;
  }
};

TEST(Planning, Explores_Then_Commits_To_Fastest, false) {
  struct P : Planning_System<Fake_Executor> {
    Fake_Executor& exec() { return executor; }
  } planner;
  planner.set_tests_until_converge(2);
  Dummy_Params params(nullptr, 7);
  std::string order;
  for (int i = 0; i < 10; ++i) {
    Dummy_Opts plan = planner.create_plan(params);
    order += std::to_string(plan.i);
    planner.execute(params, plan, Workspace(), Stream(nullptr));
  }
  // two passes over the variants, the second backwards, then the fastest
  CHECK_EQ(order, std::string("1233212222"));
  CHECK(planner.converged(Dummy_Key(params)));
  auto stats = planner.make_statistics();
  CHECK_EQ(stats.get_counts().at(Dummy_Key(params)).at(Dummy_Opts(2)), (size_t)6);
  CHECK_NEAR(stats.get_means().at(Dummy_Key(params)).at(Dummy_Opts(3)), 9.0, 1e-6);
}

TEST(Planning, Median_Ignores_First_Call_Penalty, false) {
  struct P : Planning_System<Fake_Executor> {
    Fake_Executor& exec() { return executor; }
  };
  // variant 2 is fastest but pays 100 ms on its first call: the mean of three samples would
  // rank it last, the median and the minimum rank it first.
  for (auto stat : {P::MEAN, P::MEDIAN, P::MINIMUM}) {
    P planner;
    planner.exec().first_call_penalty = 100.f;
    planner.exec().cost = {{1, 5.f}, {2, 2.f}, {3, 9.f}};
    planner.set_statistic(stat);
    planner.set_tests_until_converge(3);
    Dummy_Params params(nullptr, 1);
    Dummy_Opts plan;
    for (int i = 0; i < 10; ++i) {
      plan = planner.create_plan(params);
      planner.execute(params, plan, Workspace(), Stream(nullptr));
    }
    CHECK_EQ(plan.i, 2);  // all three pay the same penalty once; 2 stays fastest under each
  }
  P planner;
  planner.exec().cost = {{1, 5.f}, {2, 2.f}, {3, 9.f}};
  planner.set_statistic(P::MEDIAN);
  Dummy_Params params(nullptr, 2);
  // only variant 2 is penalised (as when it alone needs a kernel nobody has launched yet)
  for (int i = 0; i < 9; ++i) {
    Dummy_Opts plan = planner.create_plan(params);
    planner.exec().first_call_penalty = (plan.i == 2) ? 100.f : 0.f;
    planner.execute(params, plan, Workspace(), Stream(nullptr));
  }
  CHECK_EQ(planner.create_plan(params).i, 2);
}

TEST(Planning, Run_Off_Between_Close_Variants, false) {
  // Variants 1 and 2 are 2 % apart and the slower one's first samples happen to be low, as
  // timing noise makes them: after the plain exploration variant 1 looks faster.  The run-off
  // gives both more samples and the plan goes to the truly faster variant 2; variant 3, far
  // behind, gets no extra sample.  Without the run-off the outlier wins.
  struct Noisy : Executor<Dummy_Params, Dummy_Key, Dummy_Opts> {
    void warmup(Dummy_Params, Dummy_Opts, Stream) override {}
    void execute(Dummy_Params params, Dummy_Opts opts, Workspace, Stream,
                 Device_Timer::Mode = Device_Timer::ASYNCHRONOUS) override {
      Timer_Bank& bank = timer_log[Dummy_Key(params)][opts];
      float t = opts.i == 1 ? 10.2f : opts.i == 2 ? 10.0f : 14.0f;
      if (opts.i == 1 && bank.size() < 2) t = 9.9f;   // two lucky samples
      bank.append(Device_Timer(t));
    }
  };
  for (size_t extra : {(size_t)0, (size_t)4}) {
    Planning_System<Noisy> planner;
    planner.set_tests_until_converge(3);
    planner.set_refinement(extra, 0.05f);
    Dummy_Params params(nullptr, 11);
    Dummy_Opts plan;
    for (int i = 0; i < 40 && !planner.converged(Dummy_Key(params)); ++i) {
      plan = planner.create_plan(params);
      planner.execute(params, plan, Workspace(), Stream(nullptr));
    }
    plan = planner.create_plan(params);
    CHECK(planner.converged(Dummy_Key(params)));
    CHECK_EQ(plan.i, extra == 0 ? 1 : 2);
    auto counts = planner.make_statistics().get_counts().at(Dummy_Key(params));
    CHECK_EQ(counts.at(Dummy_Opts(3)), (size_t)3);
    if (extra) CHECK_EQ(counts.at(Dummy_Opts(1)), (size_t)7);
  }
  // The reference's preset: one sample each, then the plan.
  Planning_System<Fake_Executor> ref;
  ref.use_reference_defaults();
  Dummy_Params params(nullptr, 12);
  std::string order;
  for (int i = 0; i < 5; ++i) {
    Dummy_Opts plan = ref.create_plan(params);
    order += std::to_string(plan.i);
    ref.execute(params, plan, Workspace(), Stream(nullptr));
  }
  CHECK_EQ(order, std::string("12322"));
}

TEST(Planning, Run_Off_Figures_Are_Fresh_And_The_Default_Takes_Part, false) {
  // The default variant (0) is as fast as the fastest, but every exploration sample of it is
  // 8 % high (the first call of all, then calls right behind a kernel that left the clock
  // low); variant 2 is 1 % slower than it looks during the exploration.  The default's median
  // after the exploration is outside the run-off margin, its fastest sample is not: it takes
  // part, is ranked by its run-off samples like its rivals, ties with the fastest and gets the
  // plan.  Variant 3, whose samples are all far off, gets no extra sample.
  struct Opts4 {
    int i;
    Opts4(int i = 0) : i(i) {}
    operator std::string() const { return std::to_string(i); }
    static std::vector<Opts4> enumerate() { return {Opts4(0), Opts4(1), Opts4(2), Opts4(3)}; }
    bool operator<(const Opts4& o) const { return i < o.i; }
    static Opts4 default_opts() { return Opts4(0); }
    std::unique_ptr<MatrixOp<double>> form_operation(Dummy_Params) {
      return std::make_unique<Dummy_Op<double>>();
    }
  };
  struct Biased : Executor<Dummy_Params, Dummy_Key, Opts4> {
    void warmup(Dummy_Params, Opts4, Stream) override {}
    void execute(Dummy_Params params, Opts4 opts, Workspace, Stream,
                 Device_Timer::Mode = Device_Timer::ASYNCHRONOUS) override {
      Timer_Bank& bank = timer_log[Dummy_Key(params)][opts];
      const bool exploring = bank.size() < 3;
      float t = 0.f;
      switch (opts.i) {
        case 0: t = exploring ? (bank.size() == 1 ? 10.4f : 10.8f) : 10.0f; break;
        case 1: t = 10.3f; break;
        case 2: t = exploring ? 9.95f : 10.05f; break;
        default: t = 13.0f; break;
      }
      bank.append(Device_Timer(t));
    }
  };
  Planning_System<Biased> planner;   // the defaults: 3 samples, median, 6 more within 5 %
  Dummy_Params params(nullptr, 21);
  Opts4 plan;
  for (int i = 0; i < 60; ++i) {
    plan = planner.create_plan(params);
    if (planner.converged(Dummy_Key(params))) break;   // committed: nothing more to sample
    planner.execute(params, plan, Workspace(), Stream(nullptr));
  }
  CHECK(planner.converged(Dummy_Key(params)));
  CHECK_EQ(plan.i, 0);
  auto counts = planner.make_statistics().get_counts().at(Dummy_Key(params));
  CHECK_EQ(counts.at(Opts4(0)), (size_t)9);
  CHECK_EQ(counts.at(Opts4(2)), (size_t)9);
  CHECK_EQ(counts.at(Opts4(3)), (size_t)3);
  // Without the run-off the same samples commit to variant 2 at once.
  Planning_System<Biased> hasty;
  hasty.set_refinement(0, 0.0f);
  Dummy_Params again(nullptr, 22);
  for (int i = 0; i < 13; ++i) {
    plan = hasty.create_plan(again);
    hasty.execute(again, plan, Workspace(), Stream(nullptr));
  }
  CHECK(hasty.converged(Dummy_Key(again)));
  CHECK_EQ(plan.i, 2);
}

TEST(Planning, Ties_Go_To_The_Default_Then_To_The_Smallest_Workspace, false) {
  // Figures within tie_margin of the fastest count as tied.  Among tied variants the plan goes
  // to the default variant when it is one of them, else to the one that asks for the least
  // workspace; tie_margin = 0 is the bare argmin (reference planning_system.h:83-93).
  struct Opts4 {
    int i;
    Opts4(int i = 0) : i(i) {}
    operator std::string() const { return std::to_string(i); }
    static std::vector<Opts4> enumerate() { return {Opts4(0), Opts4(1), Opts4(2), Opts4(3)}; }
    bool operator<(const Opts4& o) const { return i < o.i; }
    static Opts4 default_opts() { return Opts4(0); }
    std::unique_ptr<MatrixOp<double>> form_operation(Dummy_Params) {
      return std::make_unique<Dummy_Op<double>>();
    }
  };
  struct Timed : Executor<Dummy_Params, Dummy_Key, Opts4> {
    std::map<int, float> cost;
    std::map<int, size_t> bytes;
    void warmup(Dummy_Params, Opts4, Stream) override {}
    void execute(Dummy_Params params, Opts4 opts, Workspace, Stream,
                 Device_Timer::Mode = Device_Timer::ASYNCHRONOUS) override {
      timer_log[Dummy_Key(params)][opts].append(Device_Timer(cost[opts.i]));
    }
    size_t calculate_workspace(Dummy_Params, Opts4 opts) override { return bytes[opts.i]; }
  };
  struct P : Planning_System<Timed> {
    Timed& exec() { return executor; }
  };
  auto plan_for = [](std::map<int, float> cost, std::map<int, size_t> bytes, float margin) {
    P planner;
    planner.exec().cost = cost;
    planner.exec().bytes = bytes;
    planner.set_tie_margin(margin);
    planner.set_refinement(0, 0.0f);
    Dummy_Params params(nullptr, 5);
    // a workspace large enough for every variant, so that nothing degrades
    Workspace big((char*)nullptr, (size_t)1 << 40);
    Opts4 plan;
    for (int i = 0; i < 20; ++i) {
      plan = planner.create_plan(params);
      planner.execute(params, plan, big, Stream(nullptr));
    }
    CHECK(planner.converged(Dummy_Key(params)));
    return plan.i;
  };
  // the default (0) is 0.3 % behind the fastest (2): tied, the plan is the default
  CHECK_EQ(plan_for({{0, 10.03f}, {1, 12.f}, {2, 10.0f}, {3, 10.02f}}, {{0, 0}, {1, 0}, {2, 800}, {3, 8}}, 0.005f), 0);
  // the default is 2 % behind: not tied; of the tied ones (2 and 3) the smaller workspace wins
  CHECK_EQ(plan_for({{0, 10.2f}, {1, 12.f}, {2, 10.0f}, {3, 10.02f}}, {{0, 0}, {1, 0}, {2, 800}, {3, 8}}, 0.005f), 3);
  // equal workspace: the faster of the tied ones
  CHECK_EQ(plan_for({{0, 10.2f}, {1, 12.f}, {2, 10.0f}, {3, 10.02f}}, {{0, 0}, {1, 0}, {2, 8}, {3, 8}}, 0.005f), 2);
  // nothing within the margin of the fastest: the fastest, whatever it costs in workspace
  CHECK_EQ(plan_for({{0, 11.f}, {1, 12.f}, {2, 10.0f}, {3, 10.5f}}, {{0, 0}, {1, 0}, {2, 800}, {3, 8}}, 0.005f), 2);
  // margin 0: the bare argmin
  CHECK_EQ(plan_for({{0, 10.03f}, {1, 12.f}, {2, 10.0f}, {3, 10.02f}}, {{0, 0}, {1, 0}, {2, 800}, {3, 8}}, 0.0f), 2);

  // Noisy samples: the default's median is 0.8 % behind the fastest variant's - more than the
  // margin - but both scatter by about as much, so they count as tied and the plan is the
  // default; a variant 3 % behind is not tied, however it scatters.
  struct Noisy : Executor<Dummy_Params, Dummy_Key, Opts4> {
    void warmup(Dummy_Params, Opts4, Stream) override {}
    void execute(Dummy_Params params, Opts4 opts, Workspace, Stream,
                 Device_Timer::Mode = Device_Timer::ASYNCHRONOUS) override {
      Timer_Bank& bank = timer_log[Dummy_Key(params)][opts];
      static const float wobble[9] = {0.f, 0.12f, -0.1f, 0.07f, -0.12f, 0.1f, -0.07f, 0.03f, -0.1f};
      const float base = opts.i == 0 ? 10.08f : opts.i == 1 ? 10.3f : opts.i == 2 ? 10.0f : 12.0f;
      bank.append(Device_Timer(base + wobble[bank.size() % 9]));
    }
    size_t calculate_workspace(Dummy_Params, Opts4 opts) override { return opts.i == 2 ? 4096 : 0; }
  };
  for (float margin : {0.005f, 0.0f}) {
    Planning_System<Noisy> planner;
    planner.set_tie_margin(margin);
    planner.set_refinement(6, 0.05f);
    Dummy_Params params(nullptr, 6);
    Workspace big((char*)nullptr, (size_t)1 << 40);
    Opts4 plan;
    for (int i = 0; i < 60; ++i) {
      plan = planner.create_plan(params);
      planner.execute(params, plan, big, Stream(nullptr));
    }
    CHECK(planner.converged(Dummy_Key(params)));
    CHECK_EQ(plan.i, margin > 0.0f ? 0 : 2);
  }
}

TEST(Planning, Pattern_Filter_And_Replaceable_Filter, false) {
  CHECK(glob_match("NNN??" "?/*/*", "NNNNPN/128x64/whole"));
  CHECK(!glob_match("NNN??" "?/*/*", "TNNNPN/128x64/whole"));
  CHECK(!glob_match("NNN??" "?/*/*", "NNN/128x64"));
  CHECK(glob_match("*", ""));
  CHECK(glob_match("F?/*/split", "FT/auto/split"));
  CHECK(!glob_match("F?/*/split", "FT/auto/split/512"));
  CHECK(glob_match("**x128*", "NNN/256x128"));
  CHECK(!glob_match("?", ""));
  const GEMM_Key key(gpu::BLAS_OP_N, gpu::BLAS_OP_N, 1000, 1000, 1000);
  auto f = pattern_filter<GEMM_Key, GEMM_Options_Pad_Tile>("NNN??" "?/*/*");
  CHECK_EQ(f.apply(key).size(), (size_t)(8 * 5 * 3));
  // alternatives; the default variant is always admitted
  auto g = pattern_filter<GEMM_Key, GEMM_Options_Pad_Tile>("TNN??" "?/64x64/whole,NTNNNN/*/auto");
  auto kept = g.apply(key);
  CHECK_EQ(kept.size(), (size_t)(1 + 8 + 5));
  CHECK_EQ(std::string(kept[0]), std::string("NNNNNN/auto/auto"));
  // a planner's filter can be replaced after construction
  Planning_System<Fake_Executor> planner;
  planner.set_tests_until_converge(1);
  planner.set_filter(Option_Filter<Dummy_Key, Dummy_Opts>(
      [](std::pair<Dummy_Opts, Dummy_Key> p) { return p.first.i != 2; }));
  Dummy_Params params(nullptr, 4);
  CHECK_EQ(planner.admitted(Dummy_Key(params)).size(), (size_t)2);
  Dummy_Opts plan;
  for (int i = 0; i < 5; ++i) {
    plan = planner.create_plan(params);
    planner.execute(params, plan, Workspace(), Stream(nullptr));
  }
  CHECK_EQ(plan.i, 1);
}

TEST(Planning, Filter_Restricts_Candidates, false) {
  Option_Filter<Dummy_Key, Dummy_Opts> no_two(
      [](std::pair<Dummy_Opts, Dummy_Key> p) { return p.first.i != 2; });
  Planning_System<Fake_Executor> planner(no_two);
  planner.set_tests_until_converge(1);
  Dummy_Params params(nullptr, 3);
  Dummy_Opts plan;
  for (int i = 0; i < 5; ++i) {
    plan = planner.create_plan(params);
    planner.execute(params, plan, Workspace(), Stream(nullptr));
  }
  CHECK_EQ(plan.i, 1);  // 5 ms beats 9 ms; the 2 ms variant is filtered out
}

TEST(Planning, Learned_Filter_Keeps_What_Paid_Off, false) {
  using Stats = Planner_Statistics<GEMM_Key, GEMM_Options>;
  const GEMM_Key seen(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 4096, 4096, 4096);
  const GEMM_Key seen_too(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 4000, 4200, 4100);   // same class
  Stats::Per_Variant<Stats::Samples> times;
  times[seen][GEMM_Options('N', 'N', 'N')] = {2.0f, 1.9f, 9.0f};   // median 2.0: the fastest
  times[seen][GEMM_Options('T', 'N', 'N')] = {2.1f, 2.1f, 2.1f};   // within 10 %
  times[seen][GEMM_Options('N', 'T', 'N')] = {3.0f, 3.0f, 3.0f};   // too slow here ...
  times[seen][GEMM_Options('N', 'N', 'T')] = {4.0f, 4.0f, 4.0f};   // too slow everywhere
  times[seen_too][GEMM_Options('N', 'T', 'N')] = {1.0f};           // ... but the fastest there
  times[seen_too][GEMM_Options('N', 'N', 'N')] = {1.5f};
  Stats stats(times);
  auto filter = learn_filter(stats, 0.1f);
  auto names = [&](const GEMM_Key& key) {
    std::string all;
    for (auto& o : filter.apply(key)) all += std::string(o) + " ";
    return all;
  };
  // the class of the recorded problems: the union of what came close on either
  CHECK_EQ(names(GEMM_Key(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 4096, 4096, 4096)),
           std::string("NNN NTN TNN "));
  CHECK_EQ(names(GEMM_Key(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 3500, 5000, 4096)),
           std::string("NNN NTN TNN "));
  // other flags or another size class: nothing known, everything admitted
  CHECK_EQ(filter.apply(GEMM_Key(gpu::BLAS_OP_N, gpu::BLAS_OP_N, 4096, 4096, 4096)).size(),
           (size_t)8);
  CHECK_EQ(filter.apply(GEMM_Key(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 512, 512, 512)).size(),
           (size_t)8);
  // the default variant survives even where it lost
  times[seen][GEMM_Options('N', 'N', 'N')] = {50.0f};
  times[seen_too][GEMM_Options('N', 'N', 'N')] = {50.0f};
  Stats slow_default(times);
  auto f2 = learn_filter(slow_default, 0.1f);
  std::string kept;
  for (auto& o : f2.apply(seen)) kept += std::string(o) + " ";
  CHECK_EQ(kept, std::string("NNN NTN TNN "));
  CHECK_EQ(size_bucket(2.0 * 4096.0 * 4096.0 * 4096.0), std::string("12"));
  CHECK_EQ(shape_class(seen), shape_class(seen_too));
}

TEST(Planning, Plans_Persist_Through_JSON, false) {
  Planning_System<GEMM_Executor<double>> a, b, c;
  GEMM_Key key(gpu::BLAS_OP_T, gpu::BLAS_OP_N, 64, 32, 16);
  Json stats = Json::parse(R"([{"key": {"transA":"T","transB":"N","m":64,"n":16,"k":32},
    "options": [{"option": {"transA":"N","transB":"N","transC":"N"}, "times": [3.0, 2.5, 9.0]},
                {"option": {"transA":"T","transB":"N","transC":"N"}, "times": [1.0, 1.5, 1.2]},
                {"option": {"transA":"N","transB":"T","transC":"N"}, "times": []}]}])");
  CHECK_EQ(a.load_plans(stats), (size_t)1);
  CHECK(a.converged(key));
  CHECK_EQ(std::string(a.create_plan(key)), std::string("TNN"));
  Json plans = a.plans_json();
  CHECK_EQ(plans.size(), (size_t)1);
  CHECK_EQ(b.load_plans(Json::parse(plans.dump(2))), (size_t)1);
  CHECK_EQ(std::string(b.create_plan(key)), std::string("TNN"));
  CHECK(!c.converged(key));
}

// ---------------------------------------------------------------------------------------------
// matrixop_test.cpp
// ---------------------------------------------------------------------------------------------
TEST(MatrixOp, MoveTest, true) {
  Blas_Fixture f;
  TestMatrix<double> A(10, 12, 10);
  std::unique_ptr<MatrixOp<double>> Aop = std::make_unique<NoOp<double>>(A);
  MatrixMove<double> Bop(std::move(Aop), 1.0, false, 32);
  auto dims = Bop.dims();
  CHECK_EQ(dims.ld, (size_t)32);
  TestMatrix<double> B(dims.m, dims.n, dims.ld);
  std::vector<double> before = B.host;
  ManagedWorkspace scratch(Bop.scratch_space_req_bytes());
  Bop.execute(f.handle, B.workspace(), scratch);
  B.download();
  CHECK(max_diff(A, B) == 0.0);
  bool pad_untouched = true;  // rows m..ld-1 keep what was there
  for (size_t j = 0; j < B.n; ++j)
    for (size_t i = B.m; i < B.ld; ++i)
      pad_untouched = pad_untouched && std::memcmp(&B.at(i, j), &before[j * B.ld + i], 8) == 0;
  CHECK(pad_untouched);
}

TEST(MatrixOp, MatMulTest, true) {
  Blas_Fixture f;
  const int m = 26, k = 34, n = 27;
  TestMatrix<double> A(m, k), B(k, n), C(m, n);
  {
    MatrixMult<double> mult(std::make_unique<NoOp<double>>(A), std::make_unique<NoOp<double>>(B),
                            std::make_unique<NoOp<double>>(C), false, false, 1.0, 0.0);
    CHECK_EQ(mult.output_space_req(), (size_t)0);
    ManagedWorkspace scratch(mult.scratch_space_req_bytes());
    mult.execute(f.handle, Workspace(), scratch);
    C.download();
  }
  host_gemm(A, B, C, -1.0, 1.0, false, false);
  CHECK(C.is_zero());
}

TEST(MatrixOp, MatTrsmTest, true) {
  Blas_Fixture f;
  const int m = 10, n = 12;
  for (bool side_left : {false, true})
    for (bool lower : {false, true})
      for (bool unit_diag : {false, true})
        for (bool trans : {false, true}) {
          const int mx = side_left ? m : n, nx = side_left ? n : m;
          TestMatrix<double> A(m, m), X(mx, nx), B(mx, nx);
          make_triangular(A, lower, unit_diag, 2.0, 1.0);
          X.host = B.host;
          A.upload();
          MatrixTrs<double> trs(std::make_unique<NoOp<double>>(A),
                                std::make_unique<NoOp<double>>(B), side_left, lower, trans,
                                unit_diag, 1.0);
          CHECK_EQ(trs.output_space_req(), (size_t)0);
          ManagedWorkspace scratch(trs.scratch_space_req_bytes());
          trs.execute(f.handle, Workspace(), scratch);
          B.download();
          orc_dtrsm(side_left ? ORC_LEFT : ORC_RIGHT, lower ? ORC_LOWER : ORC_UPPER,
                    trans ? ORC_OP_T : ORC_OP_N, unit_diag ? ORC_UNIT : ORC_NON_UNIT, mx, nx, 1.0,
                    A.host.data(), m, X.host.data(), mx);
          CHECK(max_diff(B, X) < 1e-10);
        }
}

TEST(MatrixOp, MatSyrkTest, true) {
  Blas_Fixture f;
  const int k = 56, n = 72;
  for (bool lower : {false, true})
    for (bool trans : {false, true}) {
      const size_t mA = trans ? k : n, nA = trans ? n : k;
      TestMatrix<double> A(mA, nA), C(n, n);
      host_gemm(A, A, C, 1.0, 0.0, trans, !trans);
      C.upload();
      MatrixSyrk<double> syrk(std::make_unique<NoOp<double>>(A), std::make_unique<NoOp<double>>(C),
                              lower, trans, -1.0, 1.0);
      CHECK_EQ(syrk.output_space_req(), (size_t)0);
      ManagedWorkspace scratch(syrk.scratch_space_req_bytes());
      syrk.execute(f.handle, Workspace(), scratch);
      C.download();
      for (int j = 0; j < n; ++j)
        for (int i = 0; i < n; ++i)
          if ((lower && i < j) || (!lower && i > j)) C.at(i, j) = 0.0;  // untouched triangle
      CHECK(C.is_zero());
    }
}

// C = 2 A^T B, then C += (-2 A^T materialised with ld padded to 8) B  ==> 0   (matrixop_test.cpp:230)
TEST(MatrixOp, TNMulTest, true) {
  Blas_Fixture f;
  const int m = 25, k = 14, n = 32;
  TestMatrix<double> A(k, m), B(k, n), C(m, n);
  std::unique_ptr<MatrixOp<double>> Cop = std::make_unique<MatrixMult<double>>(
      std::make_unique<NoOp<double>>(A), std::make_unique<NoOp<double>>(B),
      std::make_unique<NoOp<double>>(C), true, false, 2.0, 0.0);
  std::unique_ptr<MatrixOp<double>> At =
      std::make_unique<MatrixMove<double>>(std::make_unique<NoOp<double>>(A), -2.0, true, 8);
  Cop = std::make_unique<MatrixMult<double>>(std::move(At), std::make_unique<NoOp<double>>(B),
                                             std::move(Cop), false, false, 1.0, 1.0);
  CHECK_EQ(Cop->output_space_req(), (size_t)0);
  CHECK_EQ(Cop->scratch_space_req(), (size_t)(32 * 14));
  ManagedWorkspace scratch(Cop->scratch_space_req_bytes());
  Cop->execute(f.handle, Workspace(), scratch);
  C.download();
  CHECK(C.is_zero());
}

// C = 2 A^T B^T, then C += (0.5 A^T, pad 16)(-4 B^T, pad 8) ==> 0   (matrixop_test.cpp:267)
TEST(MatrixOp, TTMulTest, true) {
  Blas_Fixture f;
  const int m = 23, k = 42, n = 61;
  TestMatrix<double> A(k, m), B(n, k), C(m, n);
  std::unique_ptr<MatrixOp<double>> Cop = std::make_unique<MatrixMult<double>>(
      std::make_unique<NoOp<double>>(A), std::make_unique<NoOp<double>>(B),
      std::make_unique<NoOp<double>>(C), true, true, 2.0, 0.0);
  std::unique_ptr<MatrixOp<double>> At =
      std::make_unique<MatrixMove<double>>(std::make_unique<NoOp<double>>(A), 0.5, true, 16);
  std::unique_ptr<MatrixOp<double>> Bt =
      std::make_unique<MatrixMove<double>>(std::make_unique<NoOp<double>>(B), -4.0, true, 8);
  Cop = std::make_unique<MatrixMult<double>>(std::move(At), std::move(Bt), std::move(Cop), false,
                                             false, 1.0, 1.0);
  ManagedWorkspace scratch(Cop->scratch_space_req_bytes());
  Cop->execute(f.handle, Workspace(), scratch);
  C.download();
  CHECK(C.is_zero());
}

// The reference keeps this test commented out (matrixop_test.cpp:304-334): host-side tiling
// minus the plain product must vanish.
TEST(MatrixOp, TiledMatMulTest, true) {
  Blas_Fixture f;
  const int m = 300, k = 200, n = 260;
  for (bool ta : {false, true})
    for (bool tb : {false, true}) {
      TestMatrix<double> A(ta ? k : m, ta ? m : k), B(tb ? n : k, tb ? k : n), C(m, n);
      TiledMatrixMult<double> tiled(std::make_unique<NoOp<double>>(A),
                                    std::make_unique<NoOp<double>>(B),
                                    std::make_unique<NoOp<double>>(C), ta, tb, 1.0, 0.0, 128, 96, 64);
      tiled.execute(f.handle, Workspace(), Workspace());
      MatrixMult<double> plain(std::make_unique<NoOp<double>>(A), std::make_unique<NoOp<double>>(B),
                               std::make_unique<NoOp<double>>(C), ta, tb, -1.0, 1.0);
      plain.execute(f.handle, Workspace(), Workspace());
      C.download();
      CHECK(C.is_zero());
    }
}

// ---------------------------------------------------------------------------------------------
// executor_test.cpp
// ---------------------------------------------------------------------------------------------
template <typename T, typename Exec, typename OptsT>
static void gemm_correctness() {
  Blas_Fixture f;
  Exec exec;
  const int m = 70, n = 45, k = 62;
  for (bool ta : {false, true})
    for (bool tb : {false, true})
      for (auto& opts : OptsT::enumerate()) {
        TestMatrix<T> A(ta ? k : m, ta ? m : k), B(tb ? n : k, tb ? k : n), C(m, n);
        GEMM_Inputs<T> in(f.handle, op_of(ta), op_of(tb), A, B, C, T(1), T(0));
        ManagedWorkspace space(exec.calculate_workspace(in, opts));
        exec.execute(in, opts, space, f.s);
        C.download();
        CHECK(!C.is_zero());
        host_gemm<T>(A, B, C, T(-1), T(1), ta, tb);
        CHECK(C.is_zero());
      }
}

TEST(GEMM_Executor, Correctness_Double, true) {
  gemm_correctness<double, GEMM_Executor<double>, GEMM_Options>();
}
TEST(GEMM_Executor, Correctness_Single, true) {
  gemm_correctness<float, GEMM_Executor<float>, GEMM_Options>();
}
TEST(GEMM_Executor, Correctness_Pad_Variants, true) {
  gemm_correctness<double, GEMM_Executor_Pad<double>, GEMM_Options_Pad>();
}
TEST(GEMM_Executor, Correctness_Tile_Variants, true) {
  gemm_correctness<double, GEMM_Executor_Tile<double>, GEMM_Options_Tile>();
}

TEST(GEMM_Executor, Correctness_Fused_Variants, true) {
  gemm_correctness<double, GEMM_Executor_Fused<double>, GEMM_Options_Fused>();
  gemm_correctness<float, GEMM_Executor_Fused<float>, GEMM_Options_Fused>();
}

TEST(Fused_Variants, Spelling_Json_And_Workspace, false) {
  // "X" joins the letters of the switch that transposes the result; the fused forms ask for
  // the scratch of the untransposed variant.
  std::string all;
  for (auto& o : GEMM_Options_Fused::enumerate()) all += std::string(o) + " ";
  // "X" builds the tree of the untransposed switch, so it is not enumerated beside it ...
  CHECK_EQ(all, std::string("NNN NNT NTN NTT TNN TNT TTN TTT "));
  all.clear();
  for (auto& o : SYRK_Options_Fused::enumerate()) all += std::string(o) + " ";
  CHECK_EQ(all, std::string("FF FT TF TT "));
  all.clear();
  for (auto& o : TRSM_Options_Fused::enumerate()) all += std::string(o) + " ";
  CHECK_EQ(all, std::string("FF FT TF TT "));
  // ... but can be asked for by name and keeps its name in plan files
  CHECK_EQ(std::string(GEMM_Options_Fused::default_opts()), std::string("NNN"));
  CHECK_EQ(std::string(from_json<GEMM_Options_Fused>(to_json(GEMM_Options_Fused('T', 'N', 'X')))),
           std::string("TNX"));
  CHECK_EQ(std::string(from_json<SYRK_Options_Fused>(to_json(SYRK_Options_Fused('T', 'X')))),
           std::string("TX"));
  CHECK_EQ(std::string(from_json<TRSM_Options_Fused>(to_json(TRSM_Options_Fused('X', 'T')))),
           std::string("XT"));
  CHECK_THROWS(Fusable_Trans_Op("F"));
  GEMM_Options_Fused parsed;
  std::istringstream("TTX") >> parsed;
  CHECK_EQ(std::string(parsed), std::string("TTX"));

  const size_t m = 100, n = 80, k = 60;
  Matrix<double> A(Workspace(), m, k, m), B(Workspace(), k, n, k), C(Workspace(), m, n, m);
  GEMM_Inputs<double> in(nullptr, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, B, C, 1.0, 0.5);
  auto need = [&](const char* v) {
    std::istringstream text(v);
    GEMM_Options_Fused o;
    text >> o;
    return o.form_operation(in)->workspace_req();
  };
  CHECK_EQ(need("NNX"), (size_t)0);
  CHECK_EQ(need("NNT"), n * m);
  CHECK_EQ(need("TNX"), need("TNN"));
  CHECK_EQ(need("TTX"), k * m + n * k);
}

TEST(TRSM_Executor, Correctness_Double, true) {
  Blas_Fixture f;
  TRSM_Executor<double> trsm_exec;
  GEMM_Executor<double> gemm_exec;
  const int m = 435, n = 527;
  for (bool side_left : {false, true})
    for (bool lower : {false, true})
      for (bool unit_diag : {false, true})
        for (bool trans : {false, true})
          for (auto& opts : TRSM_Options::enumerate()) {
            TestMatrix<double> A(m, m);
            const int mx = side_left ? m : n, nx = side_left ? n : m;
            TestMatrix<double> X(mx, nx), B(mx, nx);
            // as executor_test.cpp:150-179: diagonally dominant, or unit with small off-diagonals
            make_triangular(A, lower, unit_diag, m + 1.0, unit_diag ? (double)m : 1.0);
            A.upload();
            if (side_left) {
              GEMM_Inputs<double> in(f.handle, op_of(trans), gpu::BLAS_OP_N, A, X, B, 1.0, 0.0);
              gemm_exec.execute(in, GEMM_Options(), Workspace(), f.s);
            } else {
              GEMM_Inputs<double> in(f.handle, gpu::BLAS_OP_N, op_of(trans), X, A, B, 1.0, 0.0);
              gemm_exec.execute(in, GEMM_Options(), Workspace(), f.s);
            }
            TRSM_Inputs<double> in(f.handle, side_left ? gpu::BLAS_SIDE_LEFT : gpu::BLAS_SIDE_RIGHT,
                                   fill_of(lower), op_of(trans),
                                   unit_diag ? gpu::BLAS_DIAG_UNIT : gpu::BLAS_DIAG_NON_UNIT, A, B,
                                   1.0);
            ManagedWorkspace space(trsm_exec.calculate_workspace(in, opts));
            trsm_exec.execute(in, opts, space, f.s);
            B.download();
            CHECK(max_diff(B, X) < 1e-10);
          }
}

TEST(SYRK_Executor, Correctness_Double, true) {
  Blas_Fixture f;
  SYRK_Executor<double> syrk_exec;
  GEMM_Executor<double> gemm_exec;
  const int n = 213, k = 74;
  for (bool lower : {false, true})
    for (bool trans : {false, true})
      for (auto& opts : SYRK_Options::enumerate()) {
        TestMatrix<double> C(n, n), A(trans ? k : n, trans ? n : k);
        {
          GEMM_Inputs<double> in(f.handle, op_of(trans), op_of(!trans), A, A, C, 1.0, 0.0);
          gemm_exec.execute(in, GEMM_Options(), Workspace(), f.s);
        }
        SYRK_Inputs<double> in(f.handle, fill_of(lower), op_of(trans), A, C, -1.0, 1.0);
        ManagedWorkspace space(syrk_exec.calculate_workspace(in, opts));
        syrk_exec.execute(in, opts, space, f.s);
        C.download();
        for (int j = 0; j < n; ++j)
          for (int i = 0; i < n; ++i)
            if ((lower && i < j) || (!lower && i > j)) C.at(i, j) = 0.0;
        CHECK(C.is_zero());
      }
}

TEST(Float_Executors, SYRK_And_TRSM, true) {
  Blas_Fixture f;
  const int n = 96, k = 40;
  for (auto& opts : SYRK_Options::enumerate()) {
    SYRK_Executor<float> se;
    GEMM_Executor<float> ge;
    TestMatrix<float> C(n, n), A(n, k);
    GEMM_Inputs<float> gi(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_T, A, A, C, 1.f, 0.f);
    ge.execute(gi, GEMM_Options(), Workspace(), f.s);
    SYRK_Inputs<float> si(f.handle, gpu::BLAS_FILL_MODE_LOWER, gpu::BLAS_OP_N, A, C, -1.f, 1.f);
    ManagedWorkspace space(se.calculate_workspace(si, opts));
    se.execute(si, opts, space, f.s);
    C.download();
    for (int j = 0; j < n; ++j)
      for (int i = 0; i < j; ++i) C.at(i, j) = 0.f;
    CHECK(C.is_zero());
  }
  for (auto& opts : TRSM_Options::enumerate()) {
    TRSM_Executor<float> te;
    GEMM_Executor<float> ge;
    TestMatrix<float> A(n, n), X(n, k), B(n, k);
    for (int j = 0; j < n; ++j)
      for (int i = 0; i < n; ++i) A.at(i, j) = i == j ? 2.f + std::abs(A.at(i, j)) : A.at(i, j) / n;
    A.upload();
    GEMM_Inputs<float> gi(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, X, B, 1.f, 0.f);
    // B := tril(A) X needs a triangular A on the device for the product
    TestMatrix<float> L(n, n);
    L.host = A.host;
    for (int j = 0; j < n; ++j)
      for (int i = 0; i < j; ++i) L.at(i, j) = 0.f;
    L.upload();
    GEMM_Inputs<float> gl(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_N, L, X, B, 1.f, 0.f);
    ge.execute(gl, GEMM_Options(), Workspace(), f.s);
    (void)gi;
    TRSM_Inputs<float> ti(f.handle, gpu::BLAS_SIDE_LEFT, gpu::BLAS_FILL_MODE_LOWER, gpu::BLAS_OP_N,
                          gpu::BLAS_DIAG_NON_UNIT, L, B, 1.f);
    ManagedWorkspace space(te.calculate_workspace(ti, opts));
    te.execute(ti, opts, space, f.s);
    B.download();
    X.download();
    CHECK(max_diff(B, X) < 1e-4f);
  }
}

// ---------------------------------------------------------------------------------------------
// planning_test.cpp
// ---------------------------------------------------------------------------------------------
TEST(Planning, Dummy_Planner, true) {
  Blas_Fixture f;
  Planning_System<Dummy_Executor> planner;
  const int N = 4;
  for (int i = 0; i < N; ++i) {
    Dummy_Params params(f.handle, i);
    for (auto opts : Dummy_Opts::enumerate())
      for (int j = 0; j < opts.i; ++j) planner.execute(params, opts, Workspace(), f.s);
  }
  auto stats = planner.make_statistics();
  CHECK_EQ(stats.get_counts().size(), (size_t)N);
  for (auto& [key, per_opt] : stats.get_counts()) {
    CHECK_EQ(per_opt.size(), Dummy_Opts::enumerate().size());
    for (auto& [opt, count] : per_opt) CHECK_EQ((size_t)opt.i, count);
  }
}

TEST(Planning, GEMM_Correctness, true) {
  Blas_Fixture f;
  GEMM_Planner planner;
  const int m = 23, n = 16, k = 35;
  TestMatrix<double> A(m, k), B(k, n), C(m, n);
  GEMM_Inputs<double> in(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, B, C, 1.0, 0.0);
  for (int i = 0; i < 10; ++i)
    for (auto& plan : GEMM_Options::enumerate()) {
      ManagedWorkspace space(planner.calculate_workspace(in, plan));
      planner.execute(in, plan, space, f.s);
      C.download();
      host_gemm(A, B, C, -1.0, 1.0, false, false);
      CHECK(C.is_zero());
    }
  auto stats = planner.make_statistics();
  for (auto& [opt, count] : stats.get_counts().begin()->second) CHECK_EQ(count, (size_t)10);
}

TEST(Planning, Hello_Autotune_Converges, true) {
  Blas_Fixture f;
  GEMM_Planner planner;
  const size_t m = 423, n = 125, k = 318;
  TestMatrix<double> A(m, k), B(k, n), C(m, n);
  GEMM_Inputs<double> in(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, B, C, 1.0, 0.0);
  ManagedWorkspace space(1024);
  GEMM_Options last;
  for (int i = 0; i < 200; ++i) {
    GEMM_Options plan = planner.create_plan(in);
    space.grow_to_fit<char>(planner.calculate_workspace(in, plan));
    planner.execute(in, plan, space, f.s);
    last = plan;
  }
  gpuAssert(gpu::DeviceSynchronize());
  CHECK(planner.converged(GEMM_Key(in)));
  CHECK_EQ(std::string(planner.create_plan(in)), std::string(last));
  // 8 variants x 3 samples of exploration, then the committed plan only (untimed once its
  // log is full)
  size_t total = 0;
  auto hello_stats = planner.make_statistics();
  for (auto& [opt, count] : hello_stats.get_counts().begin()->second) total += count;
  CHECK_EQ(total, (size_t)(21 + 100));  // 7 x 3 samples + the committed plan's log, capped at 100
  C.download();
  host_gemm(A, B, C, -1.0, 1.0, false, false);
  CHECK(C.is_zero());
}

TEST(Planning, Plan_Degradation, true) {
  Blas_Fixture f;
  GEMM_Planner planner;
  const size_t m = 69, n = 123, k = 42;
  TestMatrix<double> A(m, k), B(k, n), C(m, n);
  GEMM_Inputs<double> in(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, B, C, 1.0, 0.0);
  for (auto& plan : GEMM_Options::enumerate()) {
    planner.execute(in, plan, Workspace(), f.s);  // no workspace: falls back to "NNN"
    C.download();
    host_gemm(A, B, C, -1.0, 1.0, false, false);
    CHECK(C.is_zero());
  }
  auto counts = planner.make_statistics().get_counts();
  CHECK_EQ(counts.begin()->second.size(), (size_t)1);
  CHECK_EQ(counts.begin()->second.begin()->second, (size_t)8);
}

TEST(Facade, Lazy_Planners, true) {
  Blas_Fixture f;
  ::rtat::rtat facade;
  auto& gp = facade.gemm_planner<double>();
  CHECK(&gp == &facade.gemm_planner<double>());
  TestMatrix<double> A(40, 30), B(30, 20), C(40, 20);
  GEMM_Inputs<double> in(f.handle, gpu::BLAS_OP_N, gpu::BLAS_OP_N, A, B, C, 1.0, 0.0);
  gp.execute(in, GEMM_Options(), Workspace(), f.s);
  C.download();
  host_gemm(A, B, C, -1.0, 1.0, false, false);
  CHECK(C.is_zero());
  (void)facade.trsm_planner<double>();
  (void)facade.syrk_planner<float>();
}

TEST(Harness, Exhaustive_And_Autotune_Reports, true) {
  Json problems = Json::parse(R"([{"transA":"T","transB":"N","m":96,"n":80,"k":64,"beta":0.5,"ld_pad":3}])");
  Test_Harness<Planning_System<GEMM_Executor<double>>> harness(problems);
  Json report = harness.run_exhaustive(2);
  CHECK_EQ(report.size(), (size_t)1);
  CHECK_EQ(report[0]["options"].size(), (size_t)8);
  for (const Json& o : report[0]["options"]) CHECK_EQ(o["times"].size(), (size_t)2);
  CHECK(report[0]["key"] == Json::parse(R"({"transA":"T","transB":"N","m":96,"n":80,"k":64})"));
  Json tuned = harness.run_autotune(40);
  size_t total = 0;
  for (const Json& o : tuned[0]["options"]) total += o["times"].size();
  CHECK_EQ(total, (size_t)40);
  Test_Harness<Planning_System<TRSM_Executor<double>>> th(Json::parse(
      R"([{"side":"Left","uplo":"Lower","trans":"N","diag":"Non-Unit","m":200,"n":64}])"));
  CHECK_EQ(th.run_exhaustive(1)[0]["options"].size(), (size_t)4);
  Test_Harness<Planning_System<SYRK_Executor<double>>> sh(
      Json::parse(R"([{"uplo":"Lower","trans":"N","n":128,"k":32,"beta":1.0}])"));
  CHECK_EQ(sh.run_exhaustive(1)[0]["options"].size(), (size_t)4);
}

TEST(Planner_C_API, Gemm_Through_The_Door, true) {
  Blas_Fixture f;
  rtat_planner_t p = rtat_planner_create("gemm");
  CHECK(p != nullptr);
  CHECK(rtat_planner_create("nope") == nullptr);
  CHECK_EQ(rtat_planner_variant_count(p), 8);
  const int m = 70, n = 45, k = 62;
  TestMatrix<double> A(k, m), B(k, n), C(m, n);
  const long long ws_bytes = rtat_planner_gemm_workspace_max(p, RTAT_OP_T, RTAT_OP_N, m, n, k, k, k, m);
  CHECK_EQ(ws_bytes, (long long)8 * (k * m + n * k + n * m));
  ManagedWorkspace ws((size_t)ws_bytes);
  char chosen[32];
  for (int i = 0; i < 30; ++i) {
    C.upload();
    CHECK_EQ(rtat_planner_gemm(p, f.handle, nullptr, RTAT_OP_T, RTAT_OP_N, m, n, k, 1.0,
                               (double*)A.space, k, (double*)B.space, k, 0.0, (double*)C.space, m,
                               (char*)ws, (size_t)ws_bytes, chosen, sizeof chosen), 0);
  }
  f.s.synchronize();
  C.download();
  host_gemm(A, B, C, -1.0, 1.0, true, false);
  CHECK(C.is_zero());
  Json plans = Json::parse(rtat_planner_plans_json(p));
  CHECK_EQ(plans.size(), (size_t)1);
  CHECK_EQ(std::string(from_json<GEMM_Options>(plans[0]["plan"])), std::string(chosen));
  CHECK(rtat_planner_gemm(p, f.handle, "bogus", RTAT_OP_T, RTAT_OP_N, m, n, k, 1.0,
                          (double*)A.space, k, (double*)B.space, k, 0.0, (double*)C.space, m,
                          nullptr, 0, nullptr, 0) < 0);
  CHECK(std::strlen(rtat_planner_last_error()) > 0);
  rtat_planner_destroy(p);
}

int main(int argc, char** argv) {
  std::string mode = "all", filter;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--cpu") mode = "cpu";
    else if (a == "--gpu") mode = "gpu";
    else filter = a;
  }
  return mini::run(mode, filter);
}
