// general_matrix_multiply - command-line harness for
//   C = beta * C + alpha * op(A) * op(B),  A, B, C grouped matrices.
//
// Test infrastructure: it runs the multiplication through the C++ poplin
// layer of this build (poplin/MatMul.hpp, hence the C ABI and the gfx950
// kernels) and compares the result with a float64 model on the host, as
// PopLibs' tools/general_matrix_multiply.cpp compares a device run with
// poplibs_test::gemm::generalGroupedMatrixMultiply
// (lib/poplibs_test/GeneralMatrixMultiply.cpp:89-160).  Options carry that
// tool's names (tools/general_matrix_multiply.cpp:131-228); the data ranges
// (A in [-4,4], B in [-3,3], C in [-2,2], :417-419), the tolerances (:43-46,
// :253-259) and the comparison rule (lib/poplibs_test/Util.cpp:198-217,
// 316-348) are the same.  IPU-only options (tiles-per-ipu, ipus, profile,
// show-*) are accepted and ignored.
//   exit 0 = match, 1 = mismatch or bad usage, 77 = out of device memory.
#include "poplar/OptionFlags.hpp"
#include "poplar/exceptions.hpp"
#include "poplin/MatMul.hpp"
#include "popops/ScaledAdd.hpp"
#include "poputil/exceptions.hpp"

#include "harness_util.hpp"

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <random>
#include <sstream>

namespace {

[[noreturn]] void usage(const std::string &message) {
  std::cerr << "error: " << message << "\n"
            << "usage: general_matrix_multiply --m M --k K --n N [--g G] "
               "[options]\n"
               "  see the header of tests/tools/general_matrix_multiply.cpp "
               "for the option list\n";
  std::exit(1);
}

} // namespace

int main(int argc, char **argv) try {
  using namespace poplin;
  auto opt = parseCommandLine(argc, argv);
  static const char *known[] = {
      "help", "compile-only", "device-type", "profile", "profile-dir",
      "ignore-data", "m", "k", "n", "g", "data-type", "input-type",
      "output-type", "partials-type", "fp8-format-A", "fp8-format-B",
      "fp8-scale-A", "fp8-scale-B", "fp8-format-a", "fp8-format-b",
      "fp8-scale-a", "fp8-scale-b", "alpha", "beta", "left-matrix-op",
      "right-matrix-op", "tolerance", "tiles-per-ipu",
      "available-memory-proportion", "enable-fast-reduce", "report-plan",
      "show-execution-steps", "show-var-storage", "ipus", "plan-constraints",
      "num-executions", "remap-output-tensor", "plan-constraints-file",
      "use-create-output", "pre-arrange-rhs", "seed", "timing-runs",
      // (this harness's own: arrange the right-hand side under other plan
      // constraints than the multiplication runs with, which must be refused)
      "pre-arrange-plan-constraints"};
  for (const auto &kv : opt) {
    bool ok = false;
    for (const char *k : known)
      ok = ok || kv.first == k;
    if (!ok)
      usage("unrecognised option '--" + kv.first + "'");
  }
  auto has = [&](const char *k) { return opt.count(k) != 0; };
  auto get = [&](const char *k, const std::string &dflt = "") {
    return has(k) ? opt[k] : dflt;
  };
  if (has("help"))
    usage("help requested");
  for (const char *required : {"m", "k", "n"})
    if (!has(required))
      usage(std::string("the option '--") + required + "' is required");
  const std::size_t m = std::stoul(get("m")), k = std::stoul(get("k")),
                    n = std::stoul(get("n")), g = std::stoul(get("g", "1"));
  if ((has("output-type") != has("input-type")) ||
      (has("data-type") && has("output-type")))
    throw poputil::poplibs_error("Please specify either --data-type OR "
                                 "(--input-type AND --output-type), not both.");
  poplar::Type inputType = parseType(get("data-type", "half"));
  poplar::Type outputType = inputType;
  if (has("input-type")) {
    inputType = parseType(get("input-type"));
    outputType = parseType(get("output-type"));
  }
  if (outputType == poplar::QUARTER)
    usage("the output type is half or float");
  const float alpha = std::stof(get("alpha", "1.0")),
              beta = std::stof(get("beta", "1.0"));
  auto matrixOp = [&](const char *key) {
    const std::string v = get(key, "normal");
    if (v != "normal" && v != "transpose")
      usage(std::string("--") + key + " must be normal or transpose");
    return v == "transpose";
  };
  const bool transposeA = matrixOp("left-matrix-op");
  const bool transposeB = matrixOp("right-matrix-op");
  double relTol = outputType == poplar::FLOAT ? 0.01 : 0.1;
  const double absTol = outputType == poplar::FLOAT ? 1e-6 : 1e-5;
  if (has("tolerance"))
    relTol = std::stod(get("tolerance"));
  const unsigned numExecutions = std::stoul(get("num-executions", "1"));
  const bool ignoreData = has("ignore-data");
  const bool useCreateOutput = parseBool(get("use-create-output", "false"));
  const bool preArrange = parseBool(get("pre-arrange-rhs", "false"));

  std::string planConstraints = get("plan-constraints");
  if (!planConstraints.empty() && has("plan-constraints-file"))
    throw poputil::poplibs_error("Both plan-constraints and "
                                 "plan-constraints-file were specified");
  if (has("plan-constraints-file")) {
    std::ifstream is(get("plan-constraints-file"));
    if (!is.good())
      throw poputil::poplibs_error("Plan constraints file doesn't exist");
    std::stringstream ss;
    ss << is.rdbuf();
    planConstraints = ss.str();
  }

  // tools/general_matrix_multiply.cpp:305-328
  PlanningCache cache;
  poplar::OptionFlags mmOpt;
  mmOpt.set("remapOutputTensor",
            parseBool(get("remap-output-tensor", "false")) ? "true" : "false");
  if (has("partials-type"))
    mmOpt.set("partialsType", get("partials-type"));
  if (!planConstraints.empty())
    mmOpt.set("planConstraints", planConstraints);
  if (transposeB)
    mmOpt.set("fullyConnectedPass", "TRAINING_BWD");
  else if (transposeA)
    mmOpt.set("fullyConnectedPass", "TRAINING_WU");
  if (has("available-memory-proportion"))
    mmOpt.set("availableMemoryProportion", get("available-memory-proportion"));
  mmOpt.set("enableFastReduce",
            parseBool(get("enable-fast-reduce", "false")) ? "true" : "false");

  if (has("report-plan"))
    matMulGroupedReportPlan(std::cout, inputType, outputType, {g, m, k},
                            {g, k, n}, mmOpt, &cache);
  if (has("compile-only"))
    return 0;

  QuarterMetadata mdA, mdB;
  // (--fp8-format-A and so on are the reference's spellings,
  // tools/general_matrix_multiply.cpp:166-177; the lower-case ones are kept
  // beside them)
  auto either = [&](const std::string &upper, const char *fallback) {
    std::string lower = upper;
    lower.back() = char(lower.back() - 'A' + 'a');
    return has(upper.c_str()) ? get(upper.c_str(), fallback)
                              : get(lower.c_str(), fallback);
  };
  auto format = [&](const std::string &key) {
    const std::string v = either(key, "quart152");
    if (v != "quart152" && v != "quart143")
      usage("--" + key + " must be quart152 or quart143");
    return v == "quart143" ? QuarterMetadata::Format::F143
                           : QuarterMetadata::Format::F152;
  };
  mdA.format = format("fp8-format-A");
  mdB.format = format("fp8-format-B");
  mdA.scale = std::stoi(either("fp8-scale-A", "0"));
  mdB.scale = std::stoi(either("fp8-scale-B", "0"));

  // The operands as the caller holds them: op(A) is [g][m][k], so a
  // transposed A is stored [g][k][m]; likewise B.
  const std::size_t rowsA = transposeA ? k : m, colsA = transposeA ? m : k;
  const std::size_t rowsB = transposeB ? n : k, colsB = transposeB ? k : n;
  Stream prog;
  DeviceTensor matA(inputType, {g, rowsA, colsA},
                    DeviceTensor::Layout::External,
                    g * rowsA * colsA * inputType.size());
  DeviceTensor matB(inputType, {g, rowsB, colsB},
                    DeviceTensor::Layout::External,
                    g * rowsB * colsB * inputType.size());
  matA.metadata = mdA;
  matB.metadata = mdB;
  DeviceTensor matC = createMatMulGroupedOutput(
      inputType, outputType, {g, m, k}, {g, k, n}, mmOpt, &cache);

  std::vector<double> hostA(g * m * k), hostB(g * k * n), hostC(g * m * n),
      refC(g * m * n);
  if (!ignoreData) {
    std::mt19937 engine(has("seed") ? std::stoul(get("seed")) : 5489u);
    auto fill = [&](std::vector<double> &v, double lo, double hi) {
      std::uniform_real_distribution<double> dist(lo, hi);
      for (auto &x : v)
        x = dist(engine);
    };
    fill(hostA, -4.0, 4.0);
    fill(hostB, -3.0, 3.0);
    fill(hostC, -2.0, 2.0);
    const auto bytesA = encode(hostA, inputType, mdA);
    const auto bytesB = encode(hostB, inputType, mdB);
    const auto bytesC = encode(hostC, outputType, {});
    // model: D = beta * C + alpha * op(A) * op(B) on the rounded operands
    for (std::size_t gi = 0; gi != g; ++gi)
      for (std::size_t mi = 0; mi != m; ++mi)
        for (std::size_t ni = 0; ni != n; ++ni) {
          double acc = 0;
          for (std::size_t ki = 0; ki != k; ++ki) {
            const double a = transposeA ? hostA[(gi * k + ki) * m + mi]
                                        : hostA[(gi * m + mi) * k + ki];
            const double b = transposeB ? hostB[(gi * n + ni) * k + ki]
                                        : hostB[(gi * k + ki) * n + ni];
            acc += a * b;
          }
          const std::size_t i = (gi * m + mi) * n + ni;
          refC[i] = double(beta) * hostC[i] + double(alpha) * acc;
        }
    writeTensor(matA, bytesA.data(), prog);
    writeTensor(matB, bytesB.data(), prog);
    writeTensor(matC, bytesC.data(), prog);
  }

  // op(A), op(B) as row-major tensors (PopLibs shuffles views; this copies)
  DeviceTensor lhs = transposeA ? transposeGroupedMatrix(matA, prog) : matA;
  DeviceTensor rhs = transposeB ? transposeGroupedMatrix(matB, prog) : matB;
  if (preArrange) {
    poplar::OptionFlags arrangeOpt = mmOpt;
    if (has("pre-arrange-plan-constraints"))
      arrangeOpt.set("planConstraints", get("pre-arrange-plan-constraints"));
    rhs = preArrangeMatMulGroupedInputRHS({g, m, k}, rhs, prog, outputType,
                                          arrangeOpt, &cache);
  }

  // Only the last execution's result is kept, so that repeated accumulation
  // does not saturate it (tools/general_matrix_multiply.cpp:355-372).
  DeviceTensor matD = matC;
  std::vector<uint8_t> bytesC0;
  if (numExecutions > 1 && !ignoreData) {
    bytesC0.resize(matC.bytes());
    readTensor(matC, bytesC0.data(), prog);
  }
  const int timingRuns = std::stoi(get("timing-runs", "0"));
  for (unsigned e = 0; e != numExecutions; ++e) {
    if (e && !bytesC0.empty())
      writeTensor(matD, bytesC0.data(), prog);
    if (beta == 1.0f && !useCreateOutput) {
      matMulGroupedAcc(matD, alpha, lhs, rhs, prog, mmOpt, &cache);
    } else {
      DeviceTensor product;
      if (useCreateOutput) {
        product = createMatMulGroupedOutput(inputType, outputType, {g, m, k},
                                            {g, k, n}, mmOpt, &cache);
        matMulGroupedWithOutput(lhs, rhs, product, prog, mmOpt, &cache);
      } else {
        product = matMulGrouped(lhs, rhs, prog, outputType, mmOpt, &cache);
      }
      popops::scaledAddTo(matD, beta, product, alpha, prog);
      prog.synchronize();
    }
  }
  if (timingRuns > 0) {
    DeviceTensor product = createMatMulGroupedOutput(
        inputType, outputType, {g, m, k}, {g, k, n}, mmOpt, &cache);
    matMulGroupedWithOutput(lhs, rhs, product, prog, mmOpt, &cache);
    prog.synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i != timingRuns; ++i)
      matMulGroupedWithOutput(lhs, rhs, product, prog, mmOpt, &cache);
    prog.synchronize();
    const double us =
        std::chrono::duration<double, std::micro>(
            std::chrono::steady_clock::now() - t0).count() / timingRuns;
    std::printf("matMul: %.2f us per call, %.3f TFLOP/s\n", us,
                2.0 * g * m * k * n / us * 1e-6);
  }

  bool matchesModel = true;
  if (!ignoreData) {
    std::vector<uint8_t> bytes(matD.bytes());
    readTensor(matD, bytes.data(), prog);
    const auto actual = decode(bytes, outputType);
    unsigned mismatches = 0;
    for (std::size_t i = 0; i != actual.size(); ++i) {
      const double a = actual[i], e = refC[i];
      if (std::isnan(a) || std::isnan(e) ||
          (!isClose(a, e, relTol) && std::fabs(e - a) > absTol)) {
        if (mismatches++ < 20)
          std::cerr << "mismatch on element gemm[" << i / (m * n) << ","
                    << i / n % m << "," << i % n << "]: expected=" << e
                    << " actual=" << a << " (abs=" << a - e
                    << ", rel=" << ((a / e) - 1.0) * 100.0 << "%)\n";
      }
    }
    matchesModel = mismatches == 0;
  }
  if (!matchesModel) {
    std::cerr << "Validation failed\n";
    return 1;
  }
  return 0;
} catch (const poplar::graph_memory_allocation_error &e) {
  std::cerr << "out of device memory: " << e.what() << "\n";
  return 77;
} catch (const std::exception &e) {
  std::cerr << "error: " << e.what() << "\n";
  return 1;
}
